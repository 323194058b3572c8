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
#include <queue>
#include <utility>
#include <vector>

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
// A slice of 128 products and more is added by the whole workgroup instead.
// ============================================================================
#ifndef COMET_SPMV_T
#define COMET_SPMV_T 256
#endif
#ifndef COMET_SPMV_PASS
#define COMET_SPMV_PASS 2048
#endif
constexpr int SPMV_T = COMET_SPMV_T;         // rows (= lanes) per workgroup
constexpr int SPMV_PASS = COMET_SPMV_PASS;   // products staged in LDS per pass

constexpr int SPMV_LONG = 128;               // a row's share of a pass from which the workgroup adds it together

__device__ inline int64_t uniform_i64(int64_t v)
{
    return ((int64_t)__builtin_amdgcn_readfirstlane((int)(v >> 32)) << 32) |
           (uint32_t)__builtin_amdgcn_readfirstlane((int)(v & 0xffffffff));
}

// The LDS a workgroup streams products through.
struct SpmvStage {
    double prod[SPMV_PASS];
    double part[SPMV_T / 64];
    int64_t long_lo[SPMV_PASS / SPMV_LONG + 1], long_hi[SPMV_PASS / SPMV_LONG + 1];
    int long_owner[SPMV_PASS / SPMV_LONG + 1], nlong;
};

// The rows [r0, rlast) of one tile, rlast - r0 <= SPMV_T, lane tid owning row r0 + tid: returns acc + the lane's row
// times x, added in the order of the row's nonzeros.  Every lane of the workgroup calls it (it holds barriers).
// P: the row pointers' type - int64 for a matrix as uploaded, int32 for the column blocks of the plan, whose row
// pointers are read again by every pass
template <typename P>
__device__ __forceinline__ double spmv_tile(SpmvStage &st, const P *__restrict__ pos, const int32_t *__restrict__ crd,
                                            const double *__restrict__ val, const double *__restrict__ x, int64_t r0,
                                            int64_t rlast, double acc)
{
    const int tid = threadIdx.x;
    const int64_t r = r0 + tid;
    const int64_t ps = (int64_t)pos[r < rlast ? r : rlast];
    const int64_t pe = (int64_t)pos[r + 1 < rlast ? r + 1 : rlast];
    const int64_t bs = uniform_i64((int64_t)pos[r0]), be = uniform_i64((int64_t)pos[rlast]);
    for (int64_t cs = bs; cs < be; cs += SPMV_PASS) {
        const int64_t ce = cs + SPMV_PASS < be ? cs + SPMV_PASS : be;
        // a pass with fewer products than SPMV_LONG holds no long share: it skips the bookkeeping and its barriers
        const bool may_be_long = ce - cs >= SPMV_LONG;
        if (may_be_long && tid == 0)
            st.nlong = 0;
        for (int64_t i = cs + tid; i < ce; i += SPMV_T)
            st.prod[i - cs] = val[i] * x[crd[i]];
        __syncthreads();
        const int64_t lo = ps > cs ? ps : cs, hi = pe < ce ? pe : ce;
        if (hi - lo < SPMV_LONG) {           // the usual case: the lane adds its row's share in order
            for (int64_t p = lo; p < hi; ++p)
                acc = acc + st.prod[p - cs];
        } else {                             // at most SPMV_PASS / SPMV_LONG lanes per pass come here
            const int slot = atomicAdd(&st.nlong, 1);
            st.long_owner[slot] = tid;
            st.long_lo[slot] = lo;
            st.long_hi[slot] = hi;
        }
        if (may_be_long) {
            // Shares of SPMV_LONG products and more are added by the whole workgroup: lane t takes products
            // t, t + 256, ..., the partial sums are added along each wavefront and then across wavefronts.
            // A fixed order, though not the row's own: such a row agrees with the sequential sum to rounding,
            // not to the bit.  The shares are of different rows, so the order in which they are taken is free.
            __syncthreads();
            const int n = __builtin_amdgcn_readfirstlane(st.nlong);
            for (int k = 0; k < n; ++k) {
                const int owner = __builtin_amdgcn_readfirstlane(st.long_owner[k]);
                const int64_t l = uniform_i64(st.long_lo[k]), h = uniform_i64(st.long_hi[k]);
                double s = 0.0;
                for (int64_t p = l + tid; p < h; p += SPMV_T)
                    s = s + st.prod[p - cs];
                for (int d = 32; d > 0; d >>= 1)
                    s = s + __shfl_down(s, d, 64);
                if ((tid & 63) == 0)
                    st.part[tid >> 6] = s;
                __syncthreads();
                if (tid == owner) {
                    double t = st.part[0];
                    for (int w = 1; w < SPMV_T / 64; ++w)
                        t = t + st.part[w];
                    acc = acc + t;
                }
                __syncthreads();
            }
        }
        __syncthreads();
    }
    return acc;
}

template <bool ACC, typename P>
__global__ __launch_bounds__(SPMV_T) void spmv_csr_stream(const P *__restrict__ pos,
                                                          const int32_t *__restrict__ crd,
                                                          const double *__restrict__ val,
                                                          const double *__restrict__ x,
                                                          double *__restrict__ y, int64_t nrows)
{
    __shared__ SpmvStage st;
    const int64_t r0 = (int64_t)blockIdx.x * SPMV_T;
    const int64_t r = r0 + threadIdx.x;
    const int64_t rlast = r0 + SPMV_T < nrows ? r0 + SPMV_T : nrows;
    double acc = 0.0;
    if (ACC && r < nrows)
        acc = y[r];
    acc = spmv_tile(st, pos, crd, val, x, r0, rlast, acc);
    if (r < nrows)
        y[r] = acc;
}

// All column blocks of the plan in one launch.  A workgroup owns `tiles` tiles of `tile_rows` rows (tile k of
// workgroup w is tile k * gridDim.x + w) and goes through the blocks in order, all its tiles in each; the row sums
// stay in LDS from block to block instead of going through y.  The grid is what the GPU holds at once, so all
// workgroups are in the same block at about the same time and gather from the same slice of x - nothing waits for
// that, it only keeps the slice in the L2.  A row's products are still added in the order of its nonzeros.
// (Measured on the benchmark matrix, 10^6 rows of 10 nonzeros: 0.061 ms against 0.076 ms for a launch per block.
// One visit per block and workgroup instead - its rows consecutive, two or three to a lane, the sums in registers -
// took 0.072 ms, 0.066 with the products staged 512 at a time: the workgroups then load together and add together,
// and the memory side idles while they add.)
constexpr int SPMV_MAX_BLOCKS = 16;
struct SpmvBases { int64_t v[SPMV_MAX_BLOCKS]; };
extern __shared__ double spmv_row_sums[];

template <typename P>
__global__ __launch_bounds__(SPMV_T) void spmv_csr_blocks(const P *__restrict__ bpos, const int32_t *__restrict__ bcrd,
                                                          const double *__restrict__ bval, SpmvBases base, int nb,
                                                          const double *__restrict__ x, double *__restrict__ y,
                                                          int64_t nrows, int tile_rows, int tiles, int accumulate)
{
    __shared__ SpmvStage st;
    const int tid = threadIdx.x;
    for (int k = 0; k < tiles; ++k) {
        const int64_t r = ((int64_t)k * gridDim.x + blockIdx.x) * tile_rows + tid;
        spmv_row_sums[k * SPMV_T + tid] = accumulate && tid < tile_rows && r < nrows ? y[r] : 0.0;
    }
    for (int b = 0; b < nb; ++b) {
        const P *pos = bpos + (int64_t)b * (nrows + 1);
        const int32_t *crd = bcrd + base.v[b];
        const double *val = bval + base.v[b];
        for (int k = 0; k < tiles; ++k) {
            const int64_t r0 = ((int64_t)k * gridDim.x + blockIdx.x) * tile_rows;
            if (r0 >= nrows)
                break;
            const int64_t rlast = r0 + tile_rows < nrows ? r0 + tile_rows : nrows;
            spmv_row_sums[k * SPMV_T + tid] = spmv_tile(st, pos, crd, val, x, r0, rlast, spmv_row_sums[k * SPMV_T + tid]);
        }
    }
    for (int k = 0; k < tiles; ++k) {
        const int64_t r = ((int64_t)k * gridDim.x + blockIdx.x) * tile_rows + tid;
        if (tid < tile_rows && r < nrows)
            y[r] = spmv_row_sums[k * SPMV_T + tid];
    }
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
// Measured on the 10^6 x 10^6 Poisson(10) matrix (x = 8 MB), ms per SpMV: one pass 0.115, slices of
// 4 MiB (2 passes) 0.075, 2 MiB (4 passes) 0.077, 1 MiB (8) 0.099, 512 KiB (16) 0.140.
#ifndef COMET_SPMV_SLICE_KB
#define COMET_SPMV_SLICE_KB 2048
#endif
constexpr int64_t SPMV_SLICE_BYTES = (int64_t)COMET_SPMV_SLICE_KB << 10;

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
__global__ void spmv_narrow_pos(const int64_t *__restrict__ in, int32_t *__restrict__ out, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        out[i] = (int32_t)in[i];
}

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
    // the blocks' row pointers are read by every pass: 32 bits are enough for them unless a block holds 2^31 nonzeros
    bool narrow = true;
    for (int b = 0; b < nb; ++b)
        narrow = narrow && totals[b] < (1ll << 31);
    if (narrow) {
        int32_t *bpos32 = nullptr;
        const int64_t count = (int64_t)nb * (n + 1);
        if (hipMalloc((void **)&bpos32, sizeof(int32_t) * (size_t)count) == hipSuccess) {
            spmv_narrow_pos<<<dim3((unsigned)ceil_div(count, 256)), dim3(256), 0, stream()>>>(bpos, bpos32, count);
            if (hipStreamSynchronize(stream()) == hipSuccess) {
                a->spmv_bpos32 = bpos32;
                (void)hipFree(bpos);
                bpos = nullptr;
            } else {
                (void)hipFree(bpos32);
            }
        } else {
            (void)hipGetLastError();        // an allocation that may fail: the 64-bit pointers stay in use
        }
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
    double *__restrict__ carry, const int32_t *__restrict__ rowmap)
{
    // rowmap: the matrix lists only some rows of C (row r of pos is row rowmap[r] of C); nullptr: all of them
    auto crow = [&](int64_t r) -> int64_t { return rowmap ? (int64_t)rowmap[r] : r; };
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
            C[crow(z) * ldc + col] = 0.0;

    double acc = 0.0;
    // a row that goes on past this chunk leaves its C value to the fix-up kernel
    if (ACC && !head && rend <= e && active)
        acc = C[crow(r) * ldc + col];

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
                                __builtin_nontemporal_store(acc, C + crow(r) * ldc + col);
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
                            acc = C[crow(r) * ldc + col];
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
    double *__restrict__ C, int64_t ldc, int64_t K, const double *__restrict__ carry,
    const int32_t *__restrict__ rowmap)
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
    const int64_t cr = rowmap ? (int64_t)rowmap[r] : r;
    if (ACC)
        acc = C[cr * ldc + col] + acc;
    for (int64_t c = c0 + 1; c <= chunk; ++c)
        acc = acc + cb[(c * 2) * 64 + lane];
    C[cr * ldc + col] = acc;
}

// ============================================================================
// SpMM, long rows: column sweep with the row sums in registers.
// ============================================================================
constexpr int SPMM_HW = 16;      // wavefronts per workgroup of the sweep
#ifndef COMET_SPMM_HR_BITS
#define COMET_SPMM_HR_BITS 3
#endif
#ifndef COMET_SPMM_HEAVY_MIN
#define COMET_SPMM_HEAVY_MIN 128
#endif
constexpr int SPMM_HRB = COMET_SPMM_HR_BITS;         // bits of a list entry that name the owned row
constexpr int SPMM_HR = 1 << SPMM_HRB;               // rows a wavefront can own
constexpr int SPMM_HCOLB = 20;                       // bits of a list entry for the column, counted from the first column of its XCD's range
// Workgroups of the sweep per XCD, one to a CU: all 32 CUs of an XCD when the sweep has the GPU to itself; fewer
// when the rows that are neither long nor single hold enough of the matrix to be worth running beside it - the
// chunk kernel that takes them waits on HBM, the sweep on the path from the L2 to the CU, and on the CUs the
// sweep leaves free the chunk kernel is not starved by it (inside a CU the older wavefronts of the sweep win every
// arbitration).  Measured on the benchmark matrix (ms per product): 32 and the kernels one after the other 0.329;
// side by side with 28 workgroups per XCD 0.336, 26 0.348, 25 0.355, 24 0.311, 23 0.319, 22 0.325.
constexpr int SPMM_HG_ALONE = 32, SPMM_HG_SHARED = 24;
constexpr int spmm_hbins(int g) { return g * SPMM_HW; }               // wavefronts (= row bins) per XCD
constexpr int spmm_hslots(int g) { return spmm_hbins(g) * SPMM_HR; }  // slots for partial sums per XCD
constexpr int spmm_hrows(int g) { return g * (SPMM_HW - 1) * SPMM_HR; }    // long rows the plan can hold
// Rows of middling length - too short for a register of their own over the whole sweep, long enough that eight
// partial sums cost less than fetching their rows of B from beyond the L2 - keep their sums in the LDS of the
// sweep's workgroups, 64 doubles per row and workgroup, and their entries ride in the lists of the wavefronts that
// own long rows, so they move through the columns at the sweep's pace and find their rows of B in the L2.
#ifndef COMET_SPMM_MED_MIN
#define COMET_SPMM_MED_MIN 32
#endif
constexpr int SPMM_MED_MIN_LEN = COMET_SPMM_MED_MIN;   // such a row has at least this many nonzeros
constexpr int SPMM_MSLOTS = 288;                        // sums a workgroup keeps in LDS: 144 KiB
constexpr int SPMM_HEAVY_MIN_LEN = COMET_SPMM_HEAVY_MIN;              // a long row has at least this many nonzeros
constexpr int SPMM_HCB = 32;                         // column blocks a wavefront's list is cut into

// One workgroup per (XCD x, row group g); workgroup w runs on XCD w % 8.  XCD x
// sweeps its eighth of the column range in ascending order, so a row of B is
// pulled into that XCD's L2 once and hit by every long row that uses it.  A
// wavefront owns up to SPMM_HR rows and keeps their sums in registers.  Its list
// is cut into 32 column blocks; inside a block the entries of one row follow
// each other, columns ascending, so a row is still summed in ascending column
// order, and a run of entries of one row is added into one plain register: the
// register file is indexed dynamically only where a run begins.
//
// Rows with a single nonzero ride along: the last wavefront of every workgroup
// owns no long rows; its list holds such rows, ordered by column, and it stores
// each product straight to that row of C.  It moves through the columns with
// the others, so its rows of B come out of the L2 window the long rows keep
// warm instead of being fetched from HBM one row each.  (Stores inside the
// lists of the long rows would stall them: loads and stores share one in-order
// counter, so every wait for a gather behind a store waits for that store too.)
//
// A lane owns two adjacent dense columns and a half-wavefront one row of B, so
// one load instruction fetches two rows, 16 bytes per lane: a CU takes 8-byte
// gathers out of the L2 at 23 bytes per clock however few rows are in play,
// 16-byte ones at 42 (measured with a gather-only kernel on a table of 0.3 to
// 4 MB per XCD).  The two halves take the even and the odd entries of the same
// run - runs are padded to even length by the plan, the pad carries no value -
// and their sums are added once, at the end.
//
// A wavefront holds 64 entries of its list at a time, one per lane, and hands
// them out with readlane; the next 64 are fetched while these are used.  The
// gathers go out in batches of 8 pairs (16 rows of B) and the batch is added
// before the next one is issued: a second batch in flight while the first is
// added made the sweep slower (0.205 against 0.193 ms for the long rows alone,
// 0.227 ms when the waits were made exact so that both batches really stayed in
// flight; batches of 4 or 16 pairs: 0.25 ms) - with sixteen wavefronts per CU
// the memory path is kept busy by the other wavefronts, and more requests
// queued per wavefront only lengthen the queues.
// Entry = column - first column of the XCD's range (the low 24 bits, so that the byte offset of the row of B is one
// 24-bit multiply-add on the entry as it is) | real, first-of-run, kept-in-LDS | owned row << SPMM_E_ROW.  The slot of
// a row kept in LDS is the entry's second word.
constexpr int SPMM_HP = 8;       // pairs of entries per batch of gathers
constexpr int SPMM_E_REAL = 1 << 24;           // not a pad
constexpr int SPMM_E_FIRST = 1 << 25;          // the entry opens a run of one owned row
constexpr int SPMM_E_MED = 1 << 26;            // the entry adds into a sum kept in LDS, in the slot its second word names
constexpr int SPMM_E_ROW = 27;                 // where the owned row sits
constexpr unsigned SPMM_E_COLMASK = 0xffffffu;
static_assert(SPMM_HCOLB <= 24 && SPMM_E_ROW + SPMM_HRB <= 32, "an entry is 32 bits");
constexpr int SPMM_HWL = SPMM_HW - 1;          // wavefronts of a workgroup that own long rows

// SMALL: B spans less than 4 GiB and has fewer than 2^24 rows of fewer than 2^24 bytes, so the byte offset of a
// gather is one 24-bit multiply and one add in 32 bits on top of a scalar base, instead of a 64-bit multiply.
template <bool SMALL>
__device__ inline void heavy_issue(double2 (&b)[SPMM_HP], int ents, int t0, int npairs, int half,
                                   const double *__restrict__ B, int64_t ldb, int64_t col)
{
#pragma unroll
    for (int u = 0; u < SPMM_HP; ++u) {
        const int t = t0 + u < npairs ? t0 + u : npairs - 1;     // past the end: reload the last one, never used
        const unsigned mine = (unsigned)__shfl(ents, 2 * t + half, 64);       // each half its own entry
        if constexpr (SMALL) {
            const unsigned off = __umul24(mine, (unsigned)ldb * 8u) + (unsigned)col * 8u;
            b[u] = *reinterpret_cast<const double2 *>(reinterpret_cast<const char *>(B) + off);
        } else {
            const int64_t j = (int64_t)(mine & SPMM_E_COLMASK);
            b[u] = *reinterpret_cast<const double2 *>(B + j * ldb + col);
        }
    }
}

extern __shared__ double spmm_medium_sums[];
__device__ inline void heavy_add(double (&accx)[SPMM_HR], double (&accy)[SPMM_HR], double2 &run, int &run_slot,
                                 const double2 (&b)[SPMM_HP], int ents, int slots,
                                 double vals, int t0, int npairs, int half, int sub, bool active)
{
#pragma unroll
    for (int u = 0; u < SPMM_HP; ++u) {
        if (t0 + u < npairs) {
            const int t = t0 + u;
            const int e0 = __builtin_amdgcn_readlane(ents, 2 * t);
            const bool med = (e0 & SPMM_E_MED) != 0;       // both entries of a pair are of the same kind
            if (e0 & SPMM_E_FIRST) {             // a run starts on an even entry
                accx[run_slot] = run.x;
                accy[run_slot] = run.y;
                run_slot = ((unsigned)e0 >> SPMM_E_ROW) & (SPMM_HR - 1);
                run.x = accx[run_slot];
                run.y = accy[run_slot];
            }
            const int mine = __shfl(ents, 2 * t + half, 64);
            const double v = __hiloint2double(__shfl(__double2hiint(vals), 2 * t + half, 64),
                                              __shfl(__double2loint(vals), 2 * t + half, 64));
            if (med) {
                const double px = v * b[u].x, py = v * b[u].y;
                const int slot = __shfl(slots, 2 * t + half, 64);
                // a row of middling length: its sum lives in LDS.  An add that returns nothing is issued and
                // forgotten; all entries of such a row are in this wavefront's list, in column order, and the adds
                // of one wavefront to one address are carried out in the order it issued them.
                if ((mine & SPMM_E_REAL) && active) {
                    double *sum = spmm_medium_sums + slot * 64 + 2 * sub;
                    __hip_atomic_fetch_add(sum, px, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    __hip_atomic_fetch_add(sum + 1, py, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
            } else if (mine & SPMM_E_REAL) {     // a pad carries no value
                // A branch over the lanes of a pad, not a select: two fused multiply-adds instead of two
                // multiplications, two additions and four selects (a long row's sum is to rounding in any case:
                // it is added from sixteen partial sums).
                asm volatile("" ::: "memory");
                run.x = __builtin_fma(v, b[u].x, run.x);
                run.y = __builtin_fma(v, b[u].y, run.y);
            }
        }
    }
}

typedef int spmm_v4i __attribute__((ext_vector_type(4)));
typedef double spmm_v2d __attribute__((ext_vector_type(2)));

// The list of rows with one nonzero: a stream of pairs of entries, one entry per half-wavefront; each is one
// gather of B and one store to C.  Loads and stores share one in-order counter, so the loop is built to have
// the same number of each on every path: 32 entries at a time go through a 64-entry ring in LDS that only
// this wavefront touches (fetched one turn ahead, so no wait ever reaches back past a store), every lane always
// stores - pads, idle lanes and the turns past the end of the list store to a dump row - and nothing is
// branched around.  A wait for a batch of gathers then never includes the stores issued behind it.
// NB = pairs per batch; KB = where the turn's 32 entries start in the ring.
template <bool SMALL, bool ACC, int NB, int KB>
__device__ inline void single_issue(double2 (&b)[NB], double2 (&c)[NB], const spmm_v4i *ring_half, int t,
                                    const double *__restrict__ B, int64_t ldb, const double *__restrict__ C,
                                    int64_t ldc, int64_t col)
{
#pragma unroll
    for (int u = 0; u < NB; ++u) {
        const spmm_v4i q = ring_half[(KB + 2 * (t + u)) & 63];
        const unsigned mine = (unsigned)q.x;
        if constexpr (SMALL) {
            const unsigned off = __umul24(mine, (unsigned)ldb * 8u) + (unsigned)col * 8u;
            b[u] = *reinterpret_cast<const double2 *>(reinterpret_cast<const char *>(B) + off);
        } else {
            const int64_t j = (int64_t)(mine & SPMM_E_COLMASK);
            b[u] = *reinterpret_cast<const double2 *>(B + j * ldb + col);
        }
        if constexpr (ACC)
            c[u] = *reinterpret_cast<const double2 *>(C + (int64_t)q.y * ldc + col);
    }
    __builtin_amdgcn_sched_barrier(0);       // the gathers stay in front of the stores of the other batch
}

template <bool ACC, int NB, int KB>
__device__ inline void single_store(const double2 (&b)[NB], const double2 (&c)[NB], const spmm_v4i *ring_half, int t,
                                    int64_t pair0, int64_t npairs, double *__restrict__ C, int64_t ldc, int64_t col,
                                    bool active, double *__restrict__ dump)
{
#pragma unroll
    for (int u = 0; u < NB; ++u) {
        const spmm_v4i q = ring_half[(KB + 2 * (t + u)) & 63];
        const double v = __hiloint2double(q.w, q.z);
        spmm_v2d o;
        o.x = (ACC ? c[u].x : 0.0) + v * b[u].x;
        o.y = (ACC ? c[u].y : 0.0) + v * b[u].y;
        const bool ok = pair0 + t + u < npairs && active && (q.x & SPMM_E_REAL);
        double *dst = ok ? C + (int64_t)q.y * ldc + col : dump;
        __builtin_nontemporal_store(o, reinterpret_cast<spmm_v2d *>(dst));       // C is written once, not read again
        if (u & 1)
            __builtin_amdgcn_sched_barrier(0);       // two pairs at a time: keeps the entries read ahead few
    }
}

template <bool SMALL, bool ACC>
__device__ inline void single_rows(const spmm_v4i *__restrict__ list, int64_t n, int lane, int half,
                                   const double *__restrict__ B, int64_t ldb, double *__restrict__ C, int64_t ldc,
                                   int64_t col, bool active, spmm_v4i *ring, double *__restrict__ dump)
{
    constexpr int NB = ACC ? 4 : 8;
    double2 b0[NB], b1[NB], c0[NB], c1[NB];
    const int64_t npairs = n >> 1;           // the list has an even number of entries
    const int l32 = lane & 31;
    auto fetch = [&](int64_t turn) {         // the 32 entries of a turn, one per lane of each half
        const int64_t i = turn * 32 + l32;
        return __builtin_nontemporal_load(list + (i < n ? i : n - 1));
    };
    const spmm_v4i *ring_half = ring + half;
    ring[l32] = fetch(0);
    spmm_v4i next = fetch(1);
    single_issue<SMALL, ACC, NB, 0>(b0, c0, ring_half, 0, B, ldb, C, ldc, col);
    // a turn = 16 pairs: its entries, and those of the next turn for the gathers issued ahead, are in the ring
    auto turn = [&](auto kb, int64_t k) {
        constexpr int KB = decltype(kb)::value;
        ring[((KB + 32) & 63) + l32] = next;            // turn k + 1, over the entries of turn k - 1
        next = fetch(k + 2);
        for (int t = 0; t < 16; t += 2 * NB) {
            single_issue<SMALL, ACC, NB, KB>(b1, c1, ring_half, t + NB, B, ldb, C, ldc, col);
            single_store<ACC, NB, KB>(b0, c0, ring_half, t, k * 16, npairs, C, ldc, col, active, dump);
            single_issue<SMALL, ACC, NB, KB>(b0, c0, ring_half, t + 2 * NB, B, ldb, C, ldc, col);
            single_store<ACC, NB, KB>(b1, c1, ring_half, t + NB, k * 16, npairs, C, ldc, col, active, dump);
        }
    };
    for (int64_t k = 0; k * 16 < npairs; k += 2) {
        turn(std::integral_constant<int, 0>(), k);
        turn(std::integral_constant<int, 32>(), k + 1);
    }
}

template <bool SMALL, bool ACC>
__global__ __launch_bounds__(SPMM_HW * 64) void spmm_heavy_sweep(
    const int64_t *__restrict__ seg, const HeavyEnt *__restrict__ hent, const double *__restrict__ B, int64_t ldb,
    int64_t K, double *__restrict__ partial, double *__restrict__ C, int64_t ldc, int G, int64_t xcols, int nslots,
    double *__restrict__ partial_medium)
{
    const int lane = threadIdx.x & 63, half = lane >> 5, sub = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int x = blockIdx.x & 7, g = blockIdx.x >> 3;
    B += (int64_t)x * xcols * ldb;          // the entries count columns from the first one of this XCD's range
    int64_t col = (int64_t)blockIdx.y * 64 + 2 * sub;          // K is even: a lane's two columns exist or neither
    const bool active = col < K;
    if (!active)
        col = K - 2;            // idle lanes gather a valid address and store nothing
    const int64_t bin = ((int64_t)x * G + g) * SPMM_HW + wave;
    const int64_t s = seg[bin], e = seg[bin + 1];          // both even
    const spmm_v4i *list = reinterpret_cast<const spmm_v4i *>(hent);
    if (wave == SPMM_HWL) {                   // the wavefront of the rows with one nonzero
        __shared__ spmm_v4i single_ring[64];
        if (s < e)             // this wavefront's slots of `partial` hold no row: the dump
            single_rows<SMALL, ACC>(list + s, e - s, lane, half, B, ldb, C, ldc, col, active, single_ring,
                                    partial + bin * SPMM_HR * K + col);
        return;
    }
    double accx[SPMM_HR], accy[SPMM_HR];      // two plain arrays: each is indexed through M0, a double2 array is not
#pragma unroll
    for (int r = 0; r < SPMM_HR; ++r)
        accx[r] = accy[r] = 0.0;
    // the sums in LDS whose entries this wavefront's list holds: slot mod SPMM_HWL = wavefront
    for (int sl = wave; sl < nslots; sl += SPMM_HWL)
        spmm_medium_sums[sl * 64 + lane] = 0.0;
    if (s < e) {
        double2 b[SPMM_HP];
        double2 run = make_double2(0.0, 0.0);
        int run_slot = 0;
        int cnt = (int)(e - s < 64 ? e - s : 64);
        int c_ent = 0, c_slot = 0;
        double c_val = 0.0;
        if (lane < cnt) {
            const spmm_v4i q = __builtin_nontemporal_load(list + s + lane);
            c_ent = q.x;
            c_slot = q.y;
            c_val = __hiloint2double(q.w, q.z);
        }
        heavy_issue<SMALL>(b, c_ent, 0, cnt >> 1, half, B, ldb, col);
        for (int64_t base = s; base < e; base += 64) {
            const int64_t left = e - base - 64;
            const int ncnt = (int)(left < 0 ? 0 : (left < 64 ? left : 64));
            int n_ent = 0, n_slot = 0;
            double n_val = 0.0;
            if (lane < ncnt) {
                const spmm_v4i q = __builtin_nontemporal_load(list + base + 64 + lane);
                n_ent = q.x;
                n_slot = q.y;
                n_val = __hiloint2double(q.w, q.z);
            }
            const int np = cnt >> 1;
            heavy_add(accx, accy, run, run_slot, b, c_ent, c_slot, c_val, 0, np, half, sub, active);
#pragma unroll
            for (int t0 = SPMM_HP; t0 < 32; t0 += SPMM_HP)
                if (np > t0) {
                    heavy_issue<SMALL>(b, c_ent, t0, np, half, B, ldb, col);
                    heavy_add(accx, accy, run, run_slot, b, c_ent, c_slot, c_val, t0, np, half, sub, active);
                }
            if (ncnt > 0)         // the first batch of the next 64 entries: in flight over the loop's back edge
                heavy_issue<SMALL>(b, n_ent, 0, ncnt >> 1, half, B, ldb, col);
            c_ent = n_ent;
            c_slot = n_slot;
            c_val = n_val;
            cnt = ncnt;
        }
        accx[run_slot] = run.x;
        accy[run_slot] = run.y;
    }
    {   // this wavefront's sums in LDS: one partial sum per row and XCD, like the long rows'
        const int64_t c1 = (int64_t)blockIdx.y * 64 + lane;
        double *mout = partial_medium + ((int64_t)x * G + g) * nslots * K;
        for (int sl = wave; sl < nslots; sl += SPMM_HWL)
            if (c1 < K)
                mout[(int64_t)sl * K + c1] = spmm_medium_sums[sl * 64 + lane];
    }
    // even entries + odd entries, then the lower half writes both columns
    double *out = partial + (((int64_t)x * G + g) * SPMM_HW + wave) * SPMM_HR * K;
#pragma unroll
    for (int r = 0; r < SPMM_HR; ++r) {
        const double ox = __shfl_down(accx[r], 32, 64), oy = __shfl_down(accy[r], 32, 64);
        if (active && half == 0) {
            out[(int64_t)r * K + col] = accx[r] + ox;
            out[(int64_t)r * K + col + 1] = accy[r] + oy;
        }
    }
}

// C[rows[i]][0..K) = 0
__global__ void zero_listed_rows_f64(double *__restrict__ C, const int32_t *__restrict__ rows, int64_t nlisted,
                                     int64_t K, int64_t ldc)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t total = nlisted * K, step = (int64_t)gridDim.x * blockDim.x;
    for (; i < total; i += step)
        C[(int64_t)rows[i / K] * ldc + (i % K)] = 0.0;
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


// ---------------------------------------------------------------------------
// Plan for the sweep: pick the long rows, deal them to the 512 wavefronts of an
// XCD so that every wavefront gets the same number of nonzeros, and re-store
// their nonzeros as one list per (XCD, wavefront), ordered by column.
// ---------------------------------------------------------------------------
// cnt[h * 8 + x] = nonzeros of long row h whose column lies in the range XCD x sweeps
__global__ void heavy_count(int64_t nheavy, const int32_t *__restrict__ hrow, const int64_t *__restrict__ pos,
                            const int32_t *__restrict__ crd, int64_t xcols, int32_t *__restrict__ cnt)
{
    const int64_t h = (int64_t)blockIdx.x * (blockDim.x >> 3) + (threadIdx.x >> 3);
    const int x = threadIdx.x & 7;
    if (h >= nheavy)
        return;
    const int64_t s = pos[hrow[h]], e = pos[hrow[h] + 1];
    auto first_at_least = [&](int64_t c) {
        int64_t lo = s, hi = e;
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (crd[mid] < c)
                lo = mid + 1;
            else
                hi = mid;
        }
        return lo;
    };
    cnt[h * 8 + x] = (int32_t)(first_at_least((int64_t)(x + 1) * xcols) - first_at_least((int64_t)x * xcols));
}

__global__ void heavy_make_keys(int64_t nheavy, const int32_t *__restrict__ hrow, const int32_t *__restrict__ hcode,
                                const int64_t *__restrict__ hstart, const int64_t *__restrict__ pos,
                                const int32_t *__restrict__ crd, int64_t xcols, int hbins,
                                uint64_t *__restrict__ keys, uint32_t *__restrict__ idx)
{
    const int64_t h = blockIdx.x;
    if (h >= nheavy)
        return;
    const int64_t ps = pos[hrow[h]], len = pos[hrow[h] + 1] - ps, o = hstart[h];
    for (int64_t t = threadIdx.x; t < len; t += blockDim.x) {
        const uint64_t c = (uint64_t)(uint32_t)crd[ps + t];
        const uint64_t x = c / (uint64_t)xcols;
        const uint64_t cb = (c - x * (uint64_t)xcols) * SPMM_HCB / (uint64_t)xcols;   // column block inside the range
        const uint64_t code = (uint64_t)hcode[x * nheavy + h];       // wavefront * SPMM_HR + slot on that XCD
        keys[o + t] = ((((x * hbins + (code >> SPMM_HRB)) * SPMM_HCB + cb) * (2 * SPMM_HR) +
                        (code & (SPMM_HR - 1))) << 28) | c;
        idx[o + t] = (uint32_t)(ps + t);
    }
}

// The rows with one nonzero, dealt round-robin to the last wavefronts of the workgroups of the XCD that sweeps
// their column; these wavefronts own no long rows, so their lists are simply ordered by column.
__global__ void single_make_keys(int64_t nsingle, const int32_t *__restrict__ srow, const int64_t *__restrict__ pos,
                                 const int32_t *__restrict__ crd, int64_t xcols, int groups,
                                 uint64_t *__restrict__ keys, uint32_t *__restrict__ idx)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nsingle)
        return;
    const uint64_t c = (uint64_t)(uint32_t)crd[pos[srow[i]]];
    const uint64_t x = c / (uint64_t)xcols;
    const uint64_t cb = (c - x * (uint64_t)xcols) * SPMM_HCB / (uint64_t)xcols;
    const uint64_t bin = (uint64_t)(i % groups) * SPMM_HW + SPMM_HWL;
    keys[i] = ((((x * (uint64_t)spmm_hbins(groups) + bin) * SPMM_HCB + cb) * (2 * SPMM_HR) + SPMM_HR) << 28) | c;
    idx[i] = (uint32_t)i;
}

// The rows of middling length: row m of their list is kept by workgroup m % groups of every XCD, in slot
// j = m / groups, and its entries go into the list of wavefront j % SPMM_HWL of that workgroup, behind the runs of
// the wavefront's long rows in every column block.  idx = the entry's place among all such entries.
__global__ void medium_make_keys(int64_t nmedium, const int32_t *__restrict__ mrow, const int64_t *__restrict__ mstart,
                                 const int64_t *__restrict__ pos, const int32_t *__restrict__ crd, int64_t xcols,
                                 int groups, uint64_t *__restrict__ keys, uint32_t *__restrict__ idx)
{
    const int64_t m = blockIdx.x;
    if (m >= nmedium)
        return;
    const int64_t ps = pos[mrow[m]], len = pos[mrow[m] + 1] - ps, o = mstart[m];
    const uint64_t bin = (uint64_t)(m % groups) * SPMM_HW + (uint64_t)((m / groups) % SPMM_HWL);
    for (int64_t t = threadIdx.x; t < len; t += blockDim.x) {
        const uint64_t c = (uint64_t)(uint32_t)crd[ps + t];
        const uint64_t x = c / (uint64_t)xcols;
        const uint64_t cb = (c - x * (uint64_t)xcols) * SPMM_HCB / (uint64_t)xcols;
        keys[o + t] = ((((x * (uint64_t)spmm_hbins(groups) + bin) * SPMM_HCB + cb) * (2 * SPMM_HR) + SPMM_HR + 1) << 28) | c;
        idx[o + t] = (uint32_t)(o + t);
    }
}

// first[e] = 1 where entry e of the ordered list opens a run (another row, column block or wavefront)
__global__ void heavy_mark_runs(int64_t n, const uint64_t *__restrict__ keys, int64_t *__restrict__ first)
{
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e < n)
        first[e] = (e == 0 || (keys[e - 1] >> 28) != (keys[e] >> 28)) ? 1 : 0;
}

// start[r] = first entry of run r (runs[e] = runs opened before e); start[nruns] = n
__global__ void heavy_run_starts(int64_t n, const int64_t *__restrict__ first, const int64_t *__restrict__ runs,
                                 int64_t *__restrict__ start)
{
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e < n && first[e])
        start[runs[e]] = e;
    if (e == n)
        start[runs[n]] = n;
}

__global__ void heavy_run_odd(int64_t nruns, const int64_t *__restrict__ start, int64_t *__restrict__ odd)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r < nruns)
        odd[r] = (start[r + 1] - start[r]) & 1;
}

// Writes the list with every run padded to even length: entry e of run r lands at e + (pads in front of r).
// idx is a position in val for a long row's entry, a position in srow for a row with one nonzero, and a place
// among the entries of the rows of middling length for one of those.
__global__ void heavy_fill(int64_t n, const uint64_t *__restrict__ keys, const uint32_t *__restrict__ idx,
                           const double *__restrict__ val, const int64_t *__restrict__ pos,
                           const int32_t *__restrict__ srow, int64_t nmedium, const int32_t *__restrict__ mrow,
                           const int64_t *__restrict__ mstart, int groups, const int64_t *__restrict__ first,
                           const int64_t *__restrict__ runs, const int64_t *__restrict__ start,
                           const int64_t *__restrict__ pads, int64_t xcols, HeavyEnt *__restrict__ hent)
{
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n)
        return;
    const uint64_t k = keys[e];
    const int64_t r = runs[e] + first[e] - 1;
    const int64_t p = e + pads[r];
    const bool direct = ((k >> 28) & SPMM_HR) != 0;
    const uint64_t c = k & 0xfffffffull;
    const uint32_t col = (uint32_t)(c - (c / (uint64_t)xcols) * (uint64_t)xcols);     // inside its XCD's range
    HeavyEnt out;
    if (direct && ((k >> 28) & 1)) {          // a row of middling length: which one, from the entry's place
        const int64_t at = idx[e];
        int64_t lo = 0, hi = nmedium - 1;      // the last m with mstart[m] <= at
        while (lo < hi) {
            const int64_t mid = (lo + hi + 1) >> 1;
            if (mstart[mid] <= at)
                lo = mid;
            else
                hi = mid - 1;
        }
        out.ent = (int32_t)(col | SPMM_E_REAL | SPMM_E_MED);
        out.row = (int32_t)(lo / groups);
        out.val = val[pos[mrow[lo]] + (at - mstart[lo])];
    } else if (direct) {
        out.ent = (int32_t)(col | SPMM_E_REAL);
        out.row = srow[idx[e]];
        out.val = val[pos[out.row]];
    } else {
        out.ent = (int32_t)(col | SPMM_E_REAL | (first[e] ? (uint32_t)SPMM_E_FIRST : 0u) |
                            ((uint32_t)((k >> 28) & (SPMM_HR - 1)) << SPMM_E_ROW));
        out.row = 0;
        out.val = val[idx[e]];
    }
    hent[p] = out;
    if (e + 1 == start[r + 1] && ((start[r + 1] - start[r]) & 1)) {     // last entry of a run of odd length
        out.ent &= ~(SPMM_E_REAL | SPMM_E_FIRST);      // same column (a valid address), no value
        out.val = 0.0;
        hent[p + 1] = out;
    }
}

// seg[b] = position in the padded list of the first entry whose (XCD, wavefront) number is >= b
__global__ void heavy_segments(int64_t n, const uint64_t *__restrict__ keys, const int64_t *__restrict__ runs,
                               const int64_t *__restrict__ pads, int hbins, int64_t *__restrict__ seg)
{
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b > 8 * hbins)
        return;
    int64_t lo = 0, hi = n;
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if ((int64_t)(keys[mid] >> 28) / (SPMM_HCB * 2 * SPMM_HR) < b)
            lo = mid + 1;
        else
            hi = mid;
    }
    seg[b] = lo + pads[runs[lo]];      // lo opens a run (or is n): runs[lo] is that run's number
}

__global__ void light_lengths(int64_t nlight, const int32_t *__restrict__ rowmap, const int64_t *__restrict__ pos,
                              int64_t *__restrict__ len)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r < nlight)
        len[r] = pos[rowmap[r] + 1] - pos[rowmap[r]];
}

__global__ void light_copy(int64_t nlight, const int32_t *__restrict__ rowmap, const int64_t *__restrict__ pos,
                           const int32_t *__restrict__ crd, const double *__restrict__ val,
                           const int64_t *__restrict__ lpos, int32_t *__restrict__ lcrd, double *__restrict__ lval)
{
    // one 16-lane group per row: the rows copied here are short
    const int64_t r = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 4;
    const int sub = threadIdx.x & 15;
    if (r >= nlight)
        return;
    const int64_t n = lpos[r + 1] - lpos[r], src = pos[rowmap[r]], dst = lpos[r];
    for (int64_t t = sub; t < n; t += 16) {
        lcrd[dst + t] = crd[src + t];
        lval[dst + t] = val[src + t];
    }
}

// C[row] (+)= the eight per-XCD sums of a long row, in XCD (= column) order
template <bool ACC>
__global__ __launch_bounds__(256) void spmm_heavy_combine(int64_t nheavy, const int32_t *__restrict__ hrow,
                                                          const int32_t *__restrict__ hcode,
                                                          const double *__restrict__ partial, int hslots,
                                                          int64_t nmedium, const int32_t *__restrict__ mrow, int groups,
                                                          int nslots, const double *__restrict__ partial_medium,
                                                          double *__restrict__ C, int64_t ldc, int64_t K)
{
    const int lane = threadIdx.x & 63;
    const int64_t h = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t col = (int64_t)blockIdx.y * 64 + lane;
    if (h >= nheavy + nmedium || col >= K)
        return;
    if (h >= nheavy) {          // a row of middling length: slot m / groups of workgroup m % groups of every XCD
        const int64_t m = h - nheavy, row = mrow[m];
        double acc = ACC ? C[row * ldc + col] : 0.0;
        for (int x = 0; x < 8; ++x)
            acc = acc + partial_medium[((((int64_t)x * groups + m % groups) * nslots) + m / groups) * K + col];
        C[row * ldc + col] = acc;
        return;
    }
    const int64_t row = hrow[h];
    double acc = ACC ? C[row * ldc + col] : 0.0;
    for (int x = 0; x < 8; ++x)
        acc = acc + partial[((int64_t)x * hslots + hcode[x * nheavy + h]) * K + col];
    C[row * ldc + col] = acc;
}

static Workspace g_heavy_partial, g_medium_partial;

// Launches the sweep with `lds` bytes of dynamic LDS, asking for more than the 64 KiB a kernel gets by default.
template <typename Kern, typename... Args>
static void sweep_launch(Kern kernel, dim3 grid, dim3 block, size_t lds, Args... args)
{
    if (lds > 64 * 1024)
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)lds);
    kernel<<<grid, block, lds, stream()>>>(args...);
}

static int spmm_heavy_plan(Csr *a)
{
    if (a->heavy_state != 0)
        return COMET_HIP_OK;
    a->heavy_state = 1;
    if (a->nnz < (1 << 19) || a->nnz >= (1ll << 32) || ceil_div(a->ncols, 8) >= (1ll << SPMM_HCOLB))
        return COMET_HIP_OK;        // a list entry has SPMM_HCOLB bits for the column inside an XCD's eighth
    const int64_t n = a->nrows;
    std::vector<int64_t> pos((size_t)n + 1);
    COMET_HIPCHK(hipMemcpyAsync(pos.data(), a->pos, sizeof(int64_t) * (size_t)(n + 1), hipMemcpyDeviceToHost,
                                stream()));
    COMET_HIPCHK(hipStreamSynchronize(stream()));
    std::vector<std::pair<int64_t, int32_t>> cand;       // (-length, row): sorts longest first, ties by row
    std::vector<std::pair<int64_t, int32_t>> mcand;      // the same for the rows of middling length
    // Off unless COMET_HIP_SPMM_MEDIUM is set: on the benchmark matrix it takes 0.4 GB off the traffic past the L2
    // (the rows of B these rows gather are hits) and costs time - an entry of such a row takes the sweep 11 ns of a
    // CU, the chunk kernel beside the sweep 16, but the sweep is the longer of the two: 0.343 against 0.312 ms.
    const bool medium_on = getenv("COMET_HIP_SPMM_MEDIUM") != nullptr;
    for (int64_t r = 0; r < n; ++r) {
        const int64_t len = pos[(size_t)r + 1] - pos[(size_t)r];
        if (len >= SPMM_HEAVY_MIN_LEN)
            cand.emplace_back(-len, (int32_t)r);
        else if (medium_on && len >= SPMM_MED_MIN_LEN)
            mcand.emplace_back(-len, (int32_t)r);
    }
    std::sort(cand.begin(), cand.end());
    std::sort(mcand.begin(), mcand.end());
    // How many CUs of an XCD the sweep takes: all of them, unless the rows that are neither long nor single (with
    // the sweep at full size) hold at least a sixteenth of the matrix; COMET_HIP_SPMM_GROUPS overrides.
    int G = SPMM_HG_ALONE;
    {
        int64_t long_nnz = 0, single = 0;
        for (size_t k = 0; k < cand.size() && (int64_t)k < spmm_hrows(SPMM_HG_ALONE); ++k)
            long_nnz -= cand[k].first;
        for (int64_t r = 0; r < n; ++r)
            single += pos[(size_t)r + 1] - pos[(size_t)r] == 1;
        if ((a->nnz - long_nnz - single) * 16 >= a->nnz)
            G = SPMM_HG_SHARED;
        if (const char *e = getenv("COMET_HIP_SPMM_GROUPS")) {
            const int g = atoi(e);
            if (g >= 1 && g <= SPMM_HG_ALONE)
                G = g;
        }
    }
    const int hbins = spmm_hbins(G);
    // rows of middling length: the long rows the sweep has no register for, then the rows below them, longest
    // first, as many as the workgroups have slots in LDS
    std::vector<int32_t> mrow;
    std::vector<int64_t> mstart(1, 0);
    if (medium_on) {
        for (size_t k = (size_t)spmm_hrows(G); k < cand.size() && (int64_t)mrow.size() < (int64_t)G * SPMM_MSLOTS; ++k) {
            mrow.push_back(cand[k].second);
            mstart.push_back(mstart.back() - cand[k].first);
        }
        for (size_t k = 0; k < mcand.size() && (int64_t)mrow.size() < (int64_t)G * SPMM_MSLOTS; ++k) {
            mrow.push_back(mcand[k].second);
            mstart.push_back(mstart.back() - mcand[k].first);
        }
    }
    const int64_t M = (int64_t)mrow.size(), mnnz = mstart.back();
    if ((int64_t)cand.size() > spmm_hrows(G))
        cand.resize((size_t)spmm_hrows(G));
    const int64_t H = (int64_t)cand.size();
    int64_t hnnz = 0;
    for (auto &c : cand)
        hnnz -= c.first;
    if (H == 0 || hnnz * 4 < a->nnz)
        return COMET_HIP_OK;        // the long rows hold too little of the matrix to pay for a second kernel
    std::vector<int32_t> hrow((size_t)H), hcode((size_t)(8 * H)), cnt((size_t)(8 * H));
    std::vector<int64_t> hstart((size_t)H + 1, 0);
    std::vector<char> is_long((size_t)n, 0);         // 1: long, 2: of middling length
    for (int64_t m = 0; m < M; ++m)
        is_long[(size_t)mrow[(size_t)m]] = 2;
    for (int64_t k = 0; k < H; ++k) {
        hrow[(size_t)k] = cand[(size_t)k].second;
        is_long[(size_t)hrow[(size_t)k]] = 1;
        hstart[(size_t)k + 1] = hstart[(size_t)k] - cand[(size_t)k].first;
    }
    // the other rows: one nonzero -> an entry of the sweep's lists; none -> cleared; the rest -> `light`
    std::vector<int32_t> srow, erow, lrow;
    for (int64_t r = 0; r < n; ++r) {
        const int64_t len = pos[(size_t)r + 1] - pos[(size_t)r];
        if (is_long[(size_t)r])
            continue;
        (len == 0 ? erow : len == 1 ? srow : lrow).push_back((int32_t)r);
    }
    const int64_t S = (int64_t)srow.size(), E = (int64_t)erow.size(), L = (int64_t)lrow.size();
    const int64_t nent = hnnz + S + mnnz;          // entries of the lists before padding
    int32_t *d_cnt = nullptr, *d_srow = nullptr;
    int64_t *d_hstart = nullptr, *d_len = nullptr, *d_mstart = nullptr;
    int64_t *d_first = nullptr, *d_runs = nullptr, *d_start = nullptr, *d_odd = nullptr, *d_pads = nullptr;
    uint64_t *k_in = nullptr, *k_out = nullptr;
    uint32_t *i_in = nullptr, *i_out = nullptr;
    Csr *light = new Csr();
    char *scratch = nullptr;        // everything that does not outlive the planning, in one allocation
    auto cleanup = [&](bool failed) {
        (void)hipFree(scratch);
        if (failed) {
            (void)hipFree(a->heavy_seg);
            (void)hipFree(a->heavy_ent);
            (void)hipFree(a->heavy_row);
            (void)hipFree(a->heavy_code);
            (void)hipFree(a->medium_row);
            a->medium_row = nullptr;
            (void)hipFree(a->empty_rows);
            a->heavy_seg = nullptr;
            a->heavy_ent = nullptr;
            a->heavy_row = a->heavy_code = a->empty_rows = nullptr;
            a->nempty = 0;
            light->owns = true;
            csr_release(light);
        }
    };
#define HEAVY_TRY(call)                                                                                       \
    do {                                                                                                      \
        if ((call) != hipSuccess) {                                                                           \
            cleanup(true);                                                                                    \
            return set_error(COMET_HIP_ERR_HIP, "%s failed while planning the long rows", #call);             \
        }                                                                                                     \
    } while (0)
    auto at_least_one = [](int64_t v) { return (size_t)(v > 0 ? v : 1); };
    {
        // (an allocation and its release cost about as much as a product each: fourteen arrays, one of each)
        size_t total = 0;
        const auto room = [&](size_t bytes) {
            const size_t at = total;
            total += (bytes + 255) & ~(size_t)255;
            return at;
        };
        const size_t o_cnt = room(4 * (size_t)(8 * H)), o_srow = room(4 * at_least_one(S)),
                     o_hstart = room(8 * (size_t)(H + 1)), o_mstart = room(8 * (size_t)(M + 1)),
                     o_len = room(8 * at_least_one(L)), o_kin = room(8 * (size_t)nent), o_kout = room(8 * (size_t)nent),
                     o_iin = room(4 * (size_t)nent), o_iout = room(4 * (size_t)nent), o_first = room(8 * (size_t)nent),
                     o_runs = room(8 * (size_t)(nent + 1)), o_start = room(8 * (size_t)(nent + 1)),
                     o_odd = room(8 * (size_t)nent), o_pads = room(8 * (size_t)(nent + 1));
        HEAVY_TRY(hipMalloc((void **)&scratch, total));
        d_cnt = (int32_t *)(scratch + o_cnt);
        d_srow = (int32_t *)(scratch + o_srow);
        d_hstart = (int64_t *)(scratch + o_hstart);
        d_mstart = (int64_t *)(scratch + o_mstart);
        d_len = (int64_t *)(scratch + o_len);
        k_in = (uint64_t *)(scratch + o_kin);
        k_out = (uint64_t *)(scratch + o_kout);
        i_in = (uint32_t *)(scratch + o_iin);
        i_out = (uint32_t *)(scratch + o_iout);
        d_first = (int64_t *)(scratch + o_first);
        d_runs = (int64_t *)(scratch + o_runs);
        d_start = (int64_t *)(scratch + o_start);
        d_odd = (int64_t *)(scratch + o_odd);
        d_pads = (int64_t *)(scratch + o_pads);
    }
    HEAVY_TRY(hipMalloc((void **)&a->medium_row, 4 * at_least_one(M)));
    if (M > 0)
        HEAVY_TRY(hipMemcpyAsync(a->medium_row, mrow.data(), 4 * (size_t)M, hipMemcpyHostToDevice, stream()));
    HEAVY_TRY(hipMemcpyAsync(d_mstart, mstart.data(), 8 * (size_t)(M + 1), hipMemcpyHostToDevice, stream()));
    HEAVY_TRY(hipMalloc((void **)&a->heavy_seg, 8 * (size_t)(8 * hbins + 1)));
    HEAVY_TRY(hipMalloc((void **)&a->heavy_row, 4 * (size_t)H));
    HEAVY_TRY(hipMalloc((void **)&a->heavy_code, 4 * (size_t)(8 * H)));
    HEAVY_TRY(hipMalloc((void **)&a->empty_rows, 4 * at_least_one(E)));
    HEAVY_TRY(hipMalloc((void **)&light->rowmap, 4 * at_least_one(L)));
    HEAVY_TRY(hipMemcpyAsync(a->heavy_row, hrow.data(), 4 * (size_t)H, hipMemcpyHostToDevice, stream()));
    if (S > 0)
        HEAVY_TRY(hipMemcpyAsync(d_srow, srow.data(), 4 * (size_t)S, hipMemcpyHostToDevice, stream()));
    if (E > 0)
        HEAVY_TRY(hipMemcpyAsync(a->empty_rows, erow.data(), 4 * (size_t)E, hipMemcpyHostToDevice, stream()));
    if (L > 0)
        HEAVY_TRY(hipMemcpyAsync(light->rowmap, lrow.data(), 4 * (size_t)L, hipMemcpyHostToDevice, stream()));
    HEAVY_TRY(hipMemcpyAsync(d_hstart, hstart.data(), 8 * (size_t)(H + 1), hipMemcpyHostToDevice, stream()));
    const int64_t xcols = ceil_div(a->ncols, 8);
    // Every XCD gets its own assignment of rows to wavefronts, by what the row holds in that XCD's column
    // range: longest first, each to the least loaded wavefront that still has a free slot.  Wavefronts with
    // equal lists move through the columns at the same pace, which is what keeps the rows of B they share
    // inside the L2 between uses.
    heavy_count<<<dim3((unsigned)ceil_div(H, 32)), dim3(256), 0, stream()>>>(H, a->heavy_row, a->pos, a->crd, xcols,
                                                                             d_cnt);
    HEAVY_TRY(hipMemcpyAsync(cnt.data(), d_cnt, 4 * (size_t)(8 * H), hipMemcpyDeviceToHost, stream()));
    HEAVY_TRY(hipStreamSynchronize(stream()));
    for (int x = 0; x < 8; ++x) {
        std::vector<std::pair<int32_t, int32_t>> order((size_t)H);       // (-count, row index)
        for (int64_t k = 0; k < H; ++k)
            order[(size_t)k] = {-cnt[(size_t)(k * 8 + x)], (int32_t)k};
        std::sort(order.begin(), order.end());
        // (time the wavefront needs for its list so far, wavefront).  The four wavefronts of a SIMD do not
        // run at the same speed: the older one wins every arbitration, and the measured entry rates of
        // wavefronts 0-3, 4-7, 8-11, 12-15 of a workgroup are as 1.12 : 1.05 : 0.96 : 0.87.
        static const double pace[4] = {1.0 / 1.12, 1.0 / 1.05, 1.0 / 0.96, 1.0 / 0.87};
        std::priority_queue<std::pair<double, int32_t>, std::vector<std::pair<double, int32_t>>,
                            std::greater<std::pair<double, int32_t>>> bins;
        std::vector<int32_t> used((size_t)hbins, 0);
        for (int32_t b = 0; b < hbins; ++b)
            if (b % SPMM_HW != SPMM_HWL)        // the last wavefront of a workgroup takes the rows with one nonzero
                bins.push({0.0, b});
        for (auto &o : order) {
            auto top = bins.top();
            bins.pop();
            const int32_t b = top.second;
            hcode[(size_t)(x * H + o.second)] = b * SPMM_HR + used[(size_t)b];
            if (++used[(size_t)b] < SPMM_HR)
                bins.push({top.first - o.first * pace[(b % SPMM_HW) / 4], b});
        }
    }
    HEAVY_TRY(hipMemcpyAsync(a->heavy_code, hcode.data(), 4 * (size_t)(8 * H), hipMemcpyHostToDevice, stream()));
    {
        KernelTimer t("heavy_make_keys");
        heavy_make_keys<<<dim3((unsigned)H), dim3(256), 0, stream()>>>(H, a->heavy_row, a->heavy_code, d_hstart,
                                                                       a->pos, a->crd, xcols, hbins, k_in, i_in);
        if (S > 0)
            single_make_keys<<<dim3((unsigned)ceil_div(S, 256)), dim3(256), 0, stream()>>>(
                S, d_srow, a->pos, a->crd, xcols, G, k_in + hnnz, i_in + hnnz);
        if (M > 0)
            medium_make_keys<<<dim3((unsigned)M), dim3(64), 0, stream()>>>(M, a->medium_row, d_mstart, a->pos, a->crd,
                                                                          xcols, G, k_in + hnnz + S, i_in + hnnz + S);
    }
    if (sort_pairs_u64_u32(k_in, k_out, i_in, i_out, nent, 28 + (SPMM_HRB + 1) + 5 + 12) != COMET_HIP_OK) {
        cleanup(true);
        return COMET_HIP_ERR_HIP;
    }
    // runs (entries of one row inside one column block of one wavefront's list) are padded to even length
    const dim3 per_entry((unsigned)ceil_div(nent + 1, 256));
    heavy_mark_runs<<<per_entry, dim3(256), 0, stream()>>>(nent, k_out, d_first);
    if (exclusive_scan_i64(d_first, nent, d_runs) != COMET_HIP_OK) {
        cleanup(true);
        return COMET_HIP_ERR_HIP;
    }
    int64_t nruns = 0, npads = 0;
    HEAVY_TRY(hipMemcpyAsync(&nruns, d_runs + nent, 8, hipMemcpyDeviceToHost, stream()));
    HEAVY_TRY(hipStreamSynchronize(stream()));
    heavy_run_starts<<<per_entry, dim3(256), 0, stream()>>>(nent, d_first, d_runs, d_start);
    heavy_run_odd<<<dim3((unsigned)ceil_div(nruns, 256)), dim3(256), 0, stream()>>>(nruns, d_start, d_odd);
    if (exclusive_scan_i64(d_odd, nruns, d_pads) != COMET_HIP_OK) {
        cleanup(true);
        return COMET_HIP_ERR_HIP;
    }
    HEAVY_TRY(hipMemcpyAsync(&npads, d_pads + nruns, 8, hipMemcpyDeviceToHost, stream()));
    HEAVY_TRY(hipStreamSynchronize(stream()));
    HEAVY_TRY(hipMalloc((void **)&a->heavy_ent, sizeof(HeavyEnt) * (size_t)(nent + npads)));
    {
        KernelTimer t("heavy_fill");
        heavy_fill<<<dim3((unsigned)ceil_div(nent, 256)), dim3(256), 0, stream()>>>(
            nent, k_out, i_out, a->val, a->pos, d_srow, M, a->medium_row, d_mstart, G, d_first, d_runs, d_start, d_pads,
            xcols, a->heavy_ent);
        heavy_segments<<<dim3((unsigned)ceil_div(8 * hbins + 1, 256)), dim3(256), 0, stream()>>>(
            nent, k_out, d_runs, d_pads, hbins, a->heavy_seg);
    }
    // the rows of two and more nonzeros that are not long, as a matrix of their own
    light->nrows = L;
    light->ncols = a->ncols;
    light->nnz = a->nnz - hnnz - S - mnnz;
    light->owns = true;
    HEAVY_TRY(hipMalloc((void **)&light->pos, 8 * (size_t)(L + 1)));
    HEAVY_TRY(hipMalloc((void **)&light->crd, 4 * at_least_one(light->nnz)));
    HEAVY_TRY(hipMalloc((void **)&light->val, 8 * at_least_one(light->nnz)));
    if (L > 0) {
        light_lengths<<<dim3((unsigned)ceil_div(L, 256)), dim3(256), 0, stream()>>>(L, light->rowmap, a->pos, d_len);
        if (exclusive_scan_i64(d_len, L, light->pos) != COMET_HIP_OK) {
            cleanup(true);
            return COMET_HIP_ERR_HIP;
        }
        KernelTimer t("light_copy");
        light_copy<<<dim3((unsigned)ceil_div(L * 16, 256)), dim3(256), 0, stream()>>>(
            L, light->rowmap, a->pos, a->crd, a->val, light->pos, light->crd, light->val);
    } else {
        HEAVY_TRY(hipMemsetAsync(light->pos, 0, 8, stream()));
    }
    HEAVY_TRY(hipGetLastError());
    HEAVY_TRY(hipStreamSynchronize(stream()));
#undef HEAVY_TRY
    cleanup(false);
    light->heavy_state = 1;
    a->light = light;
    a->heavy_nnz = hnnz;
    a->heavy_rows = H;
    a->heavy_groups = G;
    a->medium_rows = M;
    a->nempty = E;
    a->heavy_state = 2;
    return COMET_HIP_OK;
}

}  // namespace comet

using namespace comet;

static int spmm_chunks(Csr *a, int64_t K, const double *B, int64_t ldb, double *C, int64_t ldc, int accumulate,
                       hipStream_t on = nullptr);
static int spmv_run(Csr *a, int64_t x_dptr, int64_t y_dptr, int accumulate);
static int spmm_run(Csr *a, int64_t K, int64_t b_dptr, int64_t ldb, int64_t c_dptr, int64_t ldc, int accumulate);

extern "C" int comet_hip_spmv_csr_f64(int64_t csr, int64_t x_dptr, int64_t y_dptr, int accumulate)
{
    COMET_CHK(ensure_init());
    Csr *a = csr_from_handle(csr);
    if (!a)
        return COMET_HIP_ERR_HANDLE;
    return spmv_run(a, x_dptr, y_dptr, accumulate);
}

// The launch of spmv_csr_blocks for a matrix of nrows rows: the fewest tiles per workgroup with which the
// workgroups resident at once cover all rows, and tiles of equal size (a lane per row, at most SPMV_T).  False when
// the rows do not fit the LDS of one grid: then every block is a launch of its own.
constexpr int SPMV_MAX_TILES = 16;
static bool spmv_blocks_shape(int64_t nrows, int *grid, int *tile_rows, int *tiles)
{
    static int per_cu[SPMV_MAX_TILES + 1];       // resident workgroups per CU by tiles per workgroup; 0: not asked yet
    for (int t = 1; t <= SPMV_MAX_TILES; ++t) {
        if (per_cu[t] == 0) {
            int n = 0;
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, spmv_csr_blocks<int32_t>, SPMV_T,
                                                             sizeof(double) * SPMV_T * (size_t)t) != hipSuccess || n <= 0)
                n = -1;
            per_cu[t] = n;
        }
        if (per_cu[t] < 0)
            return false;
        const int64_t resident = (int64_t)per_cu[t] * (num_cus() > 0 ? num_cus() : 256);
        if (resident * t * SPMV_T < nrows)
            continue;
        const int64_t g = std::min<int64_t>(resident, ceil_div(nrows, (int64_t)t * 64));
        *grid = (int)g;
        *tiles = t;
        *tile_rows = (int)ceil_div(nrows, g * t);
        return true;
    }
    return false;
}

static int spmv_run(Csr *a, int64_t x_dptr, int64_t y_dptr, int accumulate)
{
    if ((a->ncols > 0 && !x_dptr) || (a->nrows > 0 && !y_dptr))
        return set_error(COMET_HIP_ERR_ARG, "null vector passed to a sparse matrix-vector product");
    if (a->nrows == 0)
        return COMET_HIP_OK;
    // The column-blocked copy costs some twenty products: a matrix multiplied once runs on its own arrays, the copy
    // is made when it is multiplied again.
    const bool plan_now = a->spmv_uses > 0 || plan_at_once();
    a->spmv_uses = a->spmv_uses < 2 ? a->spmv_uses + 1 : 2;
    if (plan_now)
        COMET_CHK(spmv_plan(a));
    const int nb = a->spmv_nb > 0 ? a->spmv_nb : 1;
    const unsigned blocks = (unsigned)ceil_div(a->nrows, SPMV_T);
    const double *x = (const double *)x_dptr;
    double *y = (double *)y_dptr;
    if (nb > 1 && a->spmv_bpos32 && getenv("COMET_HIP_SPMV_LAUNCH_PER_BLOCK") == nullptr) {
        // all column blocks in one launch, the row sums staying on chip - when the workgroups the GPU holds at once
        // have room for all rows
        int grid = 0, tile_rows = 0, tiles = 0;
        if (spmv_blocks_shape(a->nrows, &grid, &tile_rows, &tiles)) {
            SpmvBases base;
            for (int b = 0; b < nb; ++b)
                base.v[b] = a->spmv_base[b];
            KernelTimer t("spmv_csr_blocks");
            spmv_csr_blocks<int32_t><<<dim3((unsigned)grid), dim3(SPMV_T), sizeof(double) * SPMV_T * (size_t)tiles,
                                       stream()>>>(a->spmv_bpos32, a->spmv_bcrd, a->spmv_bval, base, nb, x, y,
                                                   a->nrows, tile_rows, tiles, accumulate);
            COMET_HIPCHK(hipGetLastError());
            return COMET_HIP_OK;
        }
    }
    for (int b = 0; b < nb; ++b) {
        const int32_t *crd = nb == 1 ? a->crd : a->spmv_bcrd + a->spmv_base[b];
        const double *val = nb == 1 ? a->val : a->spmv_bval + a->spmv_base[b];
        const bool acc = accumulate || b > 0;   // later passes continue the row sums the earlier ones left in y
        KernelTimer t("spmv_csr_stream");
        if (nb > 1 && a->spmv_bpos32) {
            const int32_t *pos = a->spmv_bpos32 + (int64_t)b * (a->nrows + 1);
            if (acc)
                spmv_csr_stream<true, int32_t><<<dim3(blocks), dim3(SPMV_T), 0, stream()>>>(pos, crd, val, x, y, a->nrows);
            else
                spmv_csr_stream<false, int32_t><<<dim3(blocks), dim3(SPMV_T), 0, stream()>>>(pos, crd, val, x, y, a->nrows);
        } else {
            const int64_t *pos = nb == 1 ? a->pos : a->spmv_bpos + (int64_t)b * (a->nrows + 1);
            if (acc)
                spmv_csr_stream<true, int64_t><<<dim3(blocks), dim3(SPMV_T), 0, stream()>>>(pos, crd, val, x, y, a->nrows);
            else
                spmv_csr_stream<false, int64_t><<<dim3(blocks), dim3(SPMV_T), 0, stream()>>>(pos, crd, val, x, y, a->nrows);
        }
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
    return spmm_run(a, K, b_dptr, ldb, c_dptr, ldc, accumulate);
}

static int spmm_run(Csr *a, int64_t K, int64_t b_dptr, int64_t ldb, int64_t c_dptr, int64_t ldc, int accumulate)
{
    if (K < 0 || ldb < K || ldc < K)
        return set_error(COMET_HIP_ERR_ARG, "bad K/ldb/ldc (%lld, %lld, %lld)", (long long)K, (long long)ldb,
                         (long long)ldc);
    if (K == 0 || a->nrows == 0)
        return COMET_HIP_OK;
    if (!c_dptr || (a->nnz > 0 && !b_dptr))
        return set_error(COMET_HIP_ERR_ARG, "null matrix passed to a sparse-dense matrix product");
    double *C = (double *)c_dptr;
    const double *B = (const double *)b_dptr;
    if (ceil_div(K, 64) > 65535)
        return set_error(COMET_HIP_ERR_SIZE, "K = %lld needs more than 65535 column tiles", (long long)K);
    // long rows: column sweep with the sums on chip; everything else: one wavefront per 256 nonzeros
    // (the sweep loads B and stores C sixteen bytes at a time: two columns per lane, rows aligned to that)
    const bool sweep_fits = K >= 16 && K <= 2048 && (K & 1) == 0 && (ldb & 1) == 0 && (b_dptr & 15) == 0 &&
                            (ldc & 1) == 0 && (c_dptr & 15) == 0 && getenv("COMET_SPMM_NO_SWEEP") == nullptr;
    // The plan (the long rows as per-XCD lists, the rest re-packed) costs some forty products: a matrix multiplied
    // once goes through the chunk kernel whole, the plan is made when it is multiplied again.
    const bool plan_now = a->spmm_uses > 0 || plan_at_once();
    a->spmm_uses = a->spmm_uses < 2 ? a->spmm_uses + 1 : 2;
    if (sweep_fits && plan_now)
        COMET_CHK(spmm_heavy_plan(a));
    if (a->heavy_state != 2 || !sweep_fits)
        return spmm_chunks(a, K, B, ldb, C, ldc, accumulate);
    // rows of two and more nonzeros that are not long: one wavefront per 256 nonzeros
    // with CUs left free by the sweep, the chunk kernel of the rows in between runs beside it on a second stream
    const int G = a->heavy_groups;
    const bool overlap = a->light->nnz > 0 && G < SPMM_HG_ALONE;
    if (overlap) {
        // what the chunk kernel needs from stream() - its chunk table, its carry slots - is in place before the fork
        COMET_CHK(spmm_plan(a->light));
        COMET_CHK(g_spmm_carry.ensure(
            sizeof(double) * (size_t)(ceil_div(K, 64) * a->light->spmm_nchunks * 2 * 64), false));
        COMET_CHK(aux_fork());
    } else if (a->light->nnz > 0)
        COMET_CHK(spmm_chunks(a->light, K, B, ldb, C, ldc, accumulate));
    const unsigned tiles = (unsigned)ceil_div(K, 64);
    if (!accumulate && a->nempty > 0) {
        KernelTimer t("zero_listed_rows_f64");
        const unsigned blocks = (unsigned)std::min<int64_t>(ceil_div(a->nempty * K, 256), 65536);
        zero_listed_rows_f64<<<dim3(blocks), dim3(256), 0, stream()>>>(C, a->empty_rows, a->nempty, K, ldc);
    }
    // long rows (sums on chip, left in `partial`) and rows of one nonzero (stored to C)
    COMET_CHK(g_heavy_partial.ensure(sizeof(double) * 8 * (size_t)spmm_hslots(G) * (size_t)K, false));
    double *partial = (double *)g_heavy_partial.ptr;
    // rows of middling length: ceil(rows / G) sums of 64 doubles in the LDS of every workgroup
    const int nslots = (int)ceil_div(a->medium_rows, G);
    const size_t medium_lds = sizeof(double) * 64 * (size_t)nslots;
    COMET_CHK(g_medium_partial.ensure(sizeof(double) * 8 * (size_t)G * (size_t)(nslots > 0 ? nslots : 1) * (size_t)K, false));
    double *partial_medium = (double *)g_medium_partial.ptr;
    {
        KernelTimer t("spmm_heavy_sweep");
        const bool small_b = a->ncols < (1 << 24) && ldb * 8 < (1 << 24) && a->ncols * ldb * 8 < (1ll << 32);
        const dim3 grid(8 * G, tiles), block(SPMM_HW * 64);
        if (small_b && accumulate)
            sweep_launch(spmm_heavy_sweep<true, true>, grid, block, medium_lds, a->heavy_seg, a->heavy_ent, B, ldb, K, partial, C, ldc,
                         G, ceil_div(a->ncols, 8), nslots, partial_medium);
        else if (small_b)
            sweep_launch(spmm_heavy_sweep<true, false>, grid, block, medium_lds, a->heavy_seg, a->heavy_ent, B, ldb, K, partial, C, ldc,
                         G, ceil_div(a->ncols, 8), nslots, partial_medium);
        else if (accumulate)
            sweep_launch(spmm_heavy_sweep<false, true>, grid, block, medium_lds, a->heavy_seg, a->heavy_ent, B, ldb, K, partial, C, ldc,
                         G, ceil_div(a->ncols, 8), nslots, partial_medium);
        else
            sweep_launch(spmm_heavy_sweep<false, false>, grid, block, medium_lds, a->heavy_seg, a->heavy_ent, B, ldb, K, partial, C, ldc,
                         G, ceil_div(a->ncols, 8), nslots, partial_medium);
    }
    if (overlap) {      // the rows in between, on the CUs the sweep leaves free
        COMET_CHK(spmm_chunks(a->light, K, B, ldb, C, ldc, accumulate, aux_stream()));
        COMET_CHK(aux_join());
    }
    {
        KernelTimer t("spmm_heavy_combine");
        const dim3 grid((unsigned)ceil_div(a->heavy_rows + a->medium_rows, 4), tiles);
        if (accumulate)
            spmm_heavy_combine<true><<<grid, dim3(256), 0, stream()>>>(a->heavy_rows, a->heavy_row, a->heavy_code,
                                                                       partial, spmm_hslots(G), a->medium_rows,
                                                                       a->medium_row, G, nslots, partial_medium, C, ldc, K);
        else
            spmm_heavy_combine<false><<<grid, dim3(256), 0, stream()>>>(a->heavy_rows, a->heavy_row, a->heavy_code,
                                                                        partial, spmm_hslots(G), a->medium_rows,
                                                                       a->medium_row, G, nslots, partial_medium, C, ldc, K);
    }
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}

static int spmm_chunks(Csr *a, int64_t K, const double *B, int64_t ldb, double *C, int64_t ldc, int accumulate,
                       hipStream_t on)
{
    if (!on)
        on = stream();
    const int64_t b_dptr = (int64_t)B;
    if (a->nnz == 0) {
        if (!accumulate) {
            KernelTimer t("fill_rows_f64", on);
            unsigned blocks = (unsigned)std::min<int64_t>(ceil_div(a->nrows * K, 256), 65536);
            fill_rows_f64<<<dim3(blocks), dim3(256), 0, on>>>(C, a->nrows, K, ldc, 0.0);
            COMET_HIPCHK(hipGetLastError());
        }
        return COMET_HIP_OK;
    }
    COMET_CHK(spmm_plan(a));
    const int64_t nchunks = a->spmm_nchunks;
    const int64_t tiles = ceil_div(K, 64);
    COMET_CHK(g_spmm_carry.ensure(sizeof(double) * (size_t)(tiles * nchunks * 2 * 64), false));
    double *carry = (double *)g_spmm_carry.ptr;
    const dim3 grid((unsigned)ceil_div(nchunks, SPMM_WAVES), (unsigned)tiles);
    const dim3 block(SPMM_WAVES * 64);
    {
        KernelTimer t("spmm_csr_nnzsplit", on);
        if (accumulate)
            spmm_csr_nnzsplit<true><<<grid, block, 0, on>>>(a->pos, a->crd, a->val, a->nnz, a->nrows,
                                                                  a->spmm_chunk_row, nchunks, (const double *)b_dptr,
                                                                  ldb, C, ldc, K, carry, a->rowmap);
        else
            spmm_csr_nnzsplit<false><<<grid, block, 0, on>>>(a->pos, a->crd, a->val, a->nnz, a->nrows,
                                                                   a->spmm_chunk_row, nchunks, (const double *)b_dptr,
                                                                   ldb, C, ldc, K, carry, a->rowmap);
    }
    {
        KernelTimer t("spmm_csr_fixup", on);
        if (accumulate)
            spmm_csr_fixup<true><<<grid, block, 0, on>>>(a->pos, a->nnz, a->spmm_chunk_row, nchunks, C, ldc, K,
                                                               carry, a->rowmap);
        else
            spmm_csr_fixup<false><<<grid, block, 0, on>>>(a->pos, a->nnz, a->spmm_chunk_row, nchunks, C, ldc, K,
                                                                carry, a->rowmap);
    }
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}

// ---------------------------------------------------------------------------
// Yardstick for the sweep: how fast the CUs can take rows of a dense operand out of the L2 when nothing else is
// done with them.  Every wavefront walks a list of row numbers; a half-wavefront fetches one row of 64 doubles,
// 16 bytes per lane (the sweep's load shape), sixteen loads in flight, and only sums what arrives.  Workgroup w
// (on XCD w mod 8) draws its rows from the w-mod-8-th eighth of the table, so with a table of at most 4 MiB per
// XCD every gather after the first touch is an L2 hit.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void gather_rows_bench_kernel(const int32_t *__restrict__ idx, int64_t per_wave,
                                                                 const double *__restrict__ table,
                                                                 double *__restrict__ out)
{
    const int lane = threadIdx.x & 63, half = lane >> 5, sub = lane & 31;
    const int64_t wave = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 6);
    const int32_t *my = idx + wave * per_wave;
    double2 acc = make_double2(0.0, 0.0);
    for (int64_t i = 0; i < per_wave; i += 32) {
        double2 b[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const int64_t j = my[i + 2 * u + half];
            b[u] = *reinterpret_cast<const double2 *>(table + j * 64 + sub * 2);
        }
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            acc.x += b[u].x;
            acc.y += b[u].y;
        }
    }
    out[wave * 64 + lane] = acc.x + acc.y;
}

// idx[w * per_wave + i]: row of `table` (rows of 64 doubles) that wavefront w fetches i-th; 16 wavefronts per
// workgroup, `workgroups` workgroups; per_wave a multiple of 32; out holds workgroups * 1024 doubles.
extern "C" int comet_hip_gather_rows_bench(int64_t workgroups, int64_t per_wave, int64_t idx_dptr, int64_t table_dptr,
                                           int64_t table_rows, int64_t out_dptr)
{
    COMET_CHK(ensure_init());
    if (workgroups <= 0 || workgroups > 65535 || per_wave <= 0 || (per_wave & 31) || !idx_dptr || !table_dptr ||
        table_rows <= 0 || !out_dptr)
        return set_error(COMET_HIP_ERR_ARG, "bad arguments to comet_hip_gather_rows_bench");
    {
        KernelTimer t("gather_rows_bench");
        gather_rows_bench_kernel<<<dim3((unsigned)workgroups), dim3(1024), 0, stream()>>>(
            (const int32_t *)idx_dptr, per_wave, (const double *)table_dptr, (double *)out_dptr);
    }
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}

// ---------------------------------------------------------------------------
// SpMM for callers that cannot allocate (code under graph capture, serving loops that forbid hipMalloc): the
// chunk kernel and its fix-up with their scratch - the chunk -> row table and the carry slots of rows cut by a
// chunk boundary - in one array that lives in the library's image instead of in allocated workspaces.  Every
// device holds its own copy at its own address; the address is looked up once per device, when the library is
// initialised there, and host code uses that pointer, never the array's name.
// ---------------------------------------------------------------------------
constexpr int64_t SPMM_STATIC_SLOTS = 8192;      // (64-column tiles of K) x (chunks of 256 nonzeros) the array has room for
constexpr size_t SPMM_STATIC_TABLE_BYTES = sizeof(int32_t) * (size_t)SPMM_STATIC_SLOTS;
constexpr size_t SPMM_STATIC_CARRY_BYTES = sizeof(double) * 2 * 64 * (size_t)SPMM_STATIC_SLOTS;
static __device__ __align__(256) unsigned char spmm_static_scratch[SPMM_STATIC_TABLE_BYTES + SPMM_STATIC_CARRY_BYTES];
constexpr int SPMM_STATIC_MAX_DEVICES = 64;
static unsigned char *g_spmm_static_ptr[SPMM_STATIC_MAX_DEVICES];     // device address of the array, per device

namespace comet {
int spmm_static_setup(int device)
{
    if (device < 0 || device >= SPMM_STATIC_MAX_DEVICES)
        return set_error(COMET_HIP_ERR_ARG, "device %d has no slot for the static SpMM scratch", device);
    unsigned char *ptr = nullptr;
    COMET_HIPCHK(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(spmm_static_scratch)));
    g_spmm_static_ptr[device] = ptr;
    return COMET_HIP_OK;
}
}  // namespace comet

extern "C" int comet_hip_spmm_csr_f64_noalloc(int64_t csr, int64_t K, int64_t b_dptr, int64_t ldb, int64_t c_dptr,
                                              int64_t ldc, int accumulate, int64_t on_stream)
{
    // on_stream: the hipStream_t the caller wants the kernels on (a stream under graph capture, a serving loop's own
    // stream), as an integer; 0 = the library's stream, like every other entry point
    const hipStream_t on = on_stream ? (hipStream_t)on_stream : stream();
    if (!is_initialised())       // bringing the device up creates streams: the caller does that beforehand
        return set_error(COMET_HIP_ERR_ARG, "comet_hip_spmm_csr_f64_noalloc: call comet_hip_init first");
    Csr *a = csr_from_handle(csr);
    if (!a)
        return COMET_HIP_ERR_HANDLE;
    if (K < 0 || ldb < K || ldc < K)
        return set_error(COMET_HIP_ERR_ARG, "bad K/ldb/ldc (%lld, %lld, %lld)", (long long)K, (long long)ldb,
                         (long long)ldc);
    if (K == 0 || a->nrows == 0)
        return COMET_HIP_OK;
    if (!c_dptr || (a->nnz > 0 && !b_dptr))
        return set_error(COMET_HIP_ERR_ARG, "null matrix passed to a sparse-dense matrix product");
    const int64_t tiles = ceil_div(K, 64), nchunks = ceil_div(a->nnz, SPMM_CH);
    if (tiles > 65535 || tiles * nchunks > SPMM_STATIC_SLOTS)
        return set_error(COMET_HIP_ERR_SIZE,
                         "comet_hip_spmm_csr_f64_noalloc: ceil(K/64) * ceil(nnz/%d) = %lld exceeds the %lld slots of the "
                         "static scratch (nnz up to %lld at K <= 64); use comet_hip_spmm_csr_f64",
                         SPMM_CH, (long long)(tiles * nchunks), (long long)SPMM_STATIC_SLOTS,
                         (long long)(SPMM_STATIC_SLOTS * SPMM_CH));
    int device = -1;
    COMET_HIPCHK(hipGetDevice(&device));
    unsigned char *scratch = device >= 0 && device < SPMM_STATIC_MAX_DEVICES ? g_spmm_static_ptr[device] : nullptr;
    if (!scratch)
        return set_error(COMET_HIP_ERR_ARG, "the static SpMM scratch was not set up on device %d", device);
    double *C = (double *)c_dptr;
    if (a->nnz == 0) {
        if (!accumulate) {
            const unsigned blocks = (unsigned)std::min<int64_t>(ceil_div(a->nrows * K, 256), 65536);
            fill_rows_f64<<<dim3(blocks), dim3(256), 0, on>>>(C, a->nrows, K, ldc, 0.0);
            COMET_HIPCHK(hipGetLastError());
        }
        return COMET_HIP_OK;
    }
    // Every word the kernels read from the array is written earlier in the same call (the table in full, a carry
    // slot by the chunk that leaves a piece of a row in it), so nothing has to be cleared between calls.
    int32_t *chunk_row = reinterpret_cast<int32_t *>(scratch);
    double *carry = reinterpret_cast<double *>(scratch + SPMM_STATIC_TABLE_BYTES);
    spmm_chunk_rows<<<dim3((unsigned)ceil_div(nchunks, 256)), dim3(256), 0, on>>>(a->pos, a->nrows, nchunks,
                                                                                         chunk_row);
    const dim3 grid((unsigned)ceil_div(nchunks, SPMM_WAVES), (unsigned)tiles), block(SPMM_WAVES * 64);
    const double *B = (const double *)b_dptr;
    if (accumulate) {
        spmm_csr_nnzsplit<true><<<grid, block, 0, on>>>(a->pos, a->crd, a->val, a->nnz, a->nrows, chunk_row,
                                                              nchunks, B, ldb, C, ldc, K, carry, nullptr);
        spmm_csr_fixup<true><<<grid, block, 0, on>>>(a->pos, a->nnz, chunk_row, nchunks, C, ldc, K, carry,
                                                           nullptr);
    } else {
        spmm_csr_nnzsplit<false><<<grid, block, 0, on>>>(a->pos, a->crd, a->val, a->nnz, a->nrows, chunk_row,
                                                               nchunks, B, ldb, C, ldc, K, carry, nullptr);
        spmm_csr_fixup<false><<<grid, block, 0, on>>>(a->pos, a->nnz, chunk_row, nchunks, C, ldc, K, carry,
                                                            nullptr);
    }
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}

// ---------------------------------------------------------------------------
// Dense operand on the left: y[j] (+)= sum_i x[i] * B[i,j] and
// C[a,c] (+)= sum_b A[a,b] * B[b,c] with B in CSR.  The reference's nests run
// over the dense index outermost and scatter into the output
// (test/integration/ops/mult_DenseVecxCSR.ta, mult_DenseMatxCSR.ta through
// lib/Conversion/IndexTreeToSCF/IndexTreeToSCF.cpp:529-700,1247-1284), so an
// output element receives its products in ascending order of the contracted
// index.  That is the order in which the transpose of B holds them, so both
// products run as SpMV / SpMM over the transpose (built once, kept in the
// handle) and round like the reference; the dense matrix operands are turned
// by a tiled transpose on the way in and out.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void transpose2d_tile(const double *__restrict__ in, int64_t ld_in, int64_t rows,
                                                        int64_t cols, double *__restrict__ out, int64_t ld_out)
{
    __shared__ double tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;       // 32 x 8 threads
    const int64_t r0 = (int64_t)blockIdx.y * 32, c0 = (int64_t)blockIdx.x * 32;
    for (int k = ty; k < 32; k += 8)
        if (r0 + k < rows && c0 + tx < cols)
            tile[k][tx] = in[(r0 + k) * ld_in + c0 + tx];
    __syncthreads();
    for (int k = ty; k < 32; k += 8)
        if (c0 + k < cols && r0 + tx < rows)
            out[(c0 + k) * ld_out + r0 + tx] = tile[tx][k];
}

static int transpose2d(const double *in, int64_t ld_in, int64_t rows, int64_t cols, double *out, int64_t ld_out)
{
    if (rows == 0 || cols == 0)
        return COMET_HIP_OK;
    if (ceil_div(rows, 32) > 65535)
        return set_error(COMET_HIP_ERR_SIZE, "dense operand with %lld rows is too tall to turn", (long long)rows);
    KernelTimer t("transpose2d_tile");
    transpose2d_tile<<<dim3((unsigned)ceil_div(cols, 32), (unsigned)ceil_div(rows, 32)), dim3(256), 0, stream()>>>(
        in, ld_in, rows, cols, out, ld_out);
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}

static int transposed_of(Csr *b, Csr **out)
{
    if (!b->transposed) {
        b->transposed = csr_transposed_copy(b);
        if (!b->transposed)
            return COMET_HIP_ERR_HIP;
    }
    *out = b->transposed;
    return COMET_HIP_OK;
}

extern "C" int comet_hip_vecmat_csr_f64(int64_t csr, int64_t x_dptr, int64_t y_dptr, int accumulate)
{
    COMET_CHK(ensure_init());
    Csr *b = csr_from_handle(csr);
    if (!b)
        return COMET_HIP_ERR_HANDLE;
    Csr *t = nullptr;
    COMET_CHK(transposed_of(b, &t));
    return spmv_run(t, x_dptr, y_dptr, accumulate);
}

static Workspace g_left_a, g_left_c;

extern "C" int comet_hip_densemat_csr_f64(int64_t csr, int64_t M, int64_t a_dptr, int64_t lda, int64_t c_dptr,
                                          int64_t ldc, int accumulate)
{
    COMET_CHK(ensure_init());
    Csr *b = csr_from_handle(csr);
    if (!b)
        return COMET_HIP_ERR_HANDLE;
    if (M < 0 || lda < b->nrows || ldc < b->ncols)
        return set_error(COMET_HIP_ERR_ARG, "bad M/lda/ldc (%lld, %lld, %lld)", (long long)M, (long long)lda,
                         (long long)ldc);
    if (M == 0 || b->ncols == 0)
        return COMET_HIP_OK;
    if (!c_dptr || (b->nrows > 0 && !a_dptr))
        return set_error(COMET_HIP_ERR_ARG, "null matrix passed to comet_hip_densemat_csr_f64");
    Csr *t = nullptr;
    COMET_CHK(transposed_of(b, &t));
    COMET_CHK(g_left_a.ensure(sizeof(double) * (size_t)(b->nrows > 0 ? b->nrows : 1) * (size_t)M, false));
    COMET_CHK(g_left_c.ensure(sizeof(double) * (size_t)b->ncols * (size_t)M, false));
    double *at = (double *)g_left_a.ptr, *ct = (double *)g_left_c.ptr;
    COMET_CHK(transpose2d((const double *)a_dptr, lda, M, b->nrows, at, M));
    if (accumulate)
        COMET_CHK(transpose2d((const double *)c_dptr, ldc, M, b->ncols, ct, M));
    COMET_CHK(spmm_run(t, M, (int64_t)at, M, (int64_t)ct, M, accumulate));
    return transpose2d(ct, M, b->ncols, M, (double *)c_dptr, ldc);
}

// ============================================================================
// SDDMM: A = B .* (C x D), B and A sparse with one structure, C and D dense.
// The reference computes this as T = C x D followed by B .* T, and with
// --opt-fusion keeps only the entries of T that B samples
// (lib/Dialect/IndexTree/Transforms/KernelFusion.cpp:1049-1220; the test is
// test/integration/kernels/sddmm.ta).  Either way a stored entry (i, j) gets
// val * sum_k C[i,k] * D[k,j], the sum unfused and in ascending k.
// A wavefront takes 32 consecutive stored entries.  Entry by entry it loads the
// row of C and the (transposed) row of D with the lanes along k - two coalesced
// loads - and leaves the 64 products in LDS; then lane e walks along the
// products of entry e and adds them in ascending k.  D is transposed first, so
// that its "row" for a column j is contiguous; the row of every entry comes
// from a list kept in B's handle (searching pos per entry cost 80 % of the time).
// ============================================================================
#ifndef COMET_SDDMM_E
#define COMET_SDDMM_E 16
#endif
constexpr int SDDMM_E = COMET_SDDMM_E;          // entries per wavefront tile
constexpr int SDDMM_W = 4;           // wavefronts per workgroup
constexpr int SDDMM_LD = 65;         // tile row length in doubles: 64 products + 1, so a column walk hits all banks

__global__ __launch_bounds__(SDDMM_W * 64) void sddmm_kernel(int64_t nnz, const int32_t *__restrict__ entry_row,
                                                             const int32_t *__restrict__ crd,
                                                             const double *__restrict__ val,
                                                             const double *__restrict__ C, int64_t ldc,
                                                             const double *__restrict__ Dt, int64_t K,
                                                             double *__restrict__ out)
{
    __shared__ double tiles[SDDMM_W][SDDMM_E * SDDMM_LD];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    double *tile = tiles[wave];
    const int64_t base = ((int64_t)blockIdx.x * SDDMM_W + wave) * SDDMM_E;
    if (base >= nnz)
        return;
    const int cnt = (int)(nnz - base < SDDMM_E ? nnz - base : SDDMM_E);
    const int64_t p = base + (lane < cnt ? lane : cnt - 1);        // lane e < cnt owns entry base + e
    const int my_col = crd[p], my_row = entry_row[p];
    double t = 0.0;
    for (int64_t kc = 0; kc < K; kc += 64) {
        const int kn = (int)(K - kc < 64 ? K - kc : 64);
        const int64_t k = kc + (lane < kn ? lane : 0);
        double c[SDDMM_E], d[SDDMM_E];
#pragma unroll
        for (int e = 0; e < SDDMM_E; ++e) {          // past the end of a short tile: its last entry again
            const int ec = e < cnt ? e : cnt - 1;
            const int64_t j = __builtin_amdgcn_readlane(my_col, ec);
            const int64_t r = __builtin_amdgcn_readlane(my_row, ec);
            c[e] = C[r * ldc + k];
            d[e] = Dt[j * K + k];
        }
#pragma unroll
        for (int e = 0; e < SDDMM_E; ++e)
            tile[e * SDDMM_LD + lane] = c[e] * d[e];
        if (lane < cnt) {
            if (kn == 64) {
#pragma unroll 16
                for (int q = 0; q < 64; ++q)
                    t = t + tile[lane * SDDMM_LD + q];
            } else {
                for (int q = 0; q < kn; ++q)
                    t = t + tile[lane * SDDMM_LD + q];
            }
        }
    }
    if (lane < cnt)
        out[p] = val[p] * t;
}

static Workspace g_sddmm_dt;

static int sddmm_values(Csr *b, int64_t K, int64_t c_dptr, int64_t ldc, int64_t d_dptr, int64_t ldd, double *out)
{
    if (K < 0 || ldc < K || ldd < b->ncols || (b->nnz > 0 && (!out || (K > 0 && (!c_dptr || !d_dptr)))))
        return set_error(COMET_HIP_ERR_ARG, "bad operands passed to the sddmm entry point (K %lld, ldc %lld, ldd %lld)",
                         (long long)K, (long long)ldc, (long long)ldd);
    if (b->nnz == 0)
        return COMET_HIP_OK;
    if (K > 0) {
        COMET_CHK(g_sddmm_dt.ensure(sizeof(double) * (size_t)b->ncols * (size_t)K, false));
        COMET_CHK(transpose2d((const double *)d_dptr, ldd, K, b->ncols, (double *)g_sddmm_dt.ptr, K));
    }
    const int32_t *rows = nullptr;
    COMET_CHK(csr_entry_rows(b, &rows));
    {
        KernelTimer t("sddmm_kernel");
        sddmm_kernel<<<dim3((unsigned)ceil_div(b->nnz, SDDMM_W * SDDMM_E)), dim3(SDDMM_W * 64), 0, stream()>>>(
            b->nnz, rows, b->crd, b->val, (const double *)c_dptr, ldc, (const double *)g_sddmm_dt.ptr, K, out);
    }
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}

extern "C" int comet_hip_sddmm_csr_values_f64(int64_t bh, int64_t K, int64_t c_dptr, int64_t ldc, int64_t d_dptr,
                                              int64_t ldd, int64_t out_val_dptr)
{
    COMET_CHK(ensure_init());
    Csr *b = csr_from_handle(bh);
    if (!b)
        return COMET_HIP_ERR_HANDLE;
    return sddmm_values(b, K, c_dptr, ldc, d_dptr, ldd, (double *)out_val_dptr);
}

extern "C" int64_t comet_hip_sddmm_csr_f64(int64_t bh, int64_t K, int64_t c_dptr, int64_t ldc, int64_t d_dptr,
                                           int64_t ldd)
{
    if (ensure_init() != COMET_HIP_OK)
        return 0;
    Csr *b = csr_from_handle(bh);
    if (!b)
        return 0;
    Csr *a = new Csr();
    if (csr_alloc(a, b->nrows, b->ncols, b->nnz) != COMET_HIP_OK) {
        delete a;
        return 0;
    }
    bool ok = hipMemcpyAsync(a->pos, b->pos, sizeof(int64_t) * (size_t)(b->nrows + 1), hipMemcpyDeviceToDevice,
                             stream()) == hipSuccess;
    if (ok && b->nnz > 0)
        ok = hipMemcpyAsync(a->crd, b->crd, sizeof(int32_t) * (size_t)b->nnz, hipMemcpyDeviceToDevice, stream()) ==
             hipSuccess;
    if (!ok)
        set_error(COMET_HIP_ERR_HIP, "copying the structure of the sampled matrix failed");
    if (!ok || sddmm_values(b, K, c_dptr, ldc, d_dptr, ldd, a->val) != COMET_HIP_OK) {
        csr_release(a);
        return 0;
    }
    return csr_register(a);
}
