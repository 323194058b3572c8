// Input side of the sparse kernels: MatrixMarket text -> device CSR with the
// reference's read modes, the SPARSE_FILE_NAME<id> protocol of its reader
// entry points, and conversion of the other two matrix layouts its tests feed
// to SpMV/SpMM (COO and DCSR) to and from device CSR, plus CSR transposition.
//
// Text is parsed on the host; everything after that - ordering the tuples by
// (row, column) with ties in file order, dropping the entries a triangular read
// mode excludes, building the row pointers - runs on the GPU, so a matrix goes
// from file to a handle the kernels accept without a host-side CSR in between.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>

#include <exception>
#include <map>
#include <string>
#include <utility>
#include <vector>

#include "common.h"

namespace comet {

// ---------------------------------------------------------------------------
// MatrixMarket text -> unordered tuples (lib/ExecutionEngine/SparseUtils.cpp:
// 145-356): 1-based indices; a missing value reads as 1.0; the flags come from
// any line that starts with "%%" (substring tests for "symmetric", "skew",
// "array"); a symmetric file mirrors every off-diagonal entry right after the
// entry itself, negated if skew; an array file lists all rows*cols values in
// column-major order, zeros included.
// ---------------------------------------------------------------------------
struct HostCoo {
    int64_t nrows = 0, ncols = 0;
    std::vector<int32_t> row, col;
    std::vector<double> val;
};

static int parse_mtx(const char *path, HostCoo *out)
{
    FILE *f = fopen(path, "rb");
    if (!f)
        return set_error(COMET_HIP_ERR_ARG, "cannot open %s", path);
    std::string text;
    {
        char buf[1 << 16];
        size_t got;
        while ((got = fread(buf, 1, sizeof buf, f)) > 0)
            text.append(buf, got);
        fclose(f);
    }
    bool array = false, symmetric = false, skew = false, have_sizes = false;
    int64_t declared = 0, array_seen = 0;
    const char *p = text.c_str(), *end = p + text.size();
    int64_t lineno = 0;
    while (p < end) {
        const char *eol = (const char *)memchr(p, '\n', (size_t)(end - p));
        const char *next = eol ? eol + 1 : end;
        if (!eol)
            eol = end;
        ++lineno;
        std::string line(p, (size_t)(eol - p));
        p = next;
        if (!line.empty() && line[0] == '%') {
            if (line.size() > 1 && line[1] == '%') {
                symmetric = line.find("symmetric") != std::string::npos;
                skew = line.find("skew") != std::string::npos;
                array = line.find("array") != std::string::npos;
            }
            continue;
        }
        const char *l = line.c_str();
        char *t = nullptr;
        if (!have_sizes) {
            long long a = 0, b = 0, c = 0;
            const int n = sscanf(l, "%lld %lld %lld", &a, &b, &c);
            if (n < 2)
                continue;      // blank line in front of the size line
            if ((!array && n != 3) || (array && n != 2))
                return set_error(COMET_HIP_ERR_ARG, "%s:%lld: invalid size line", path, (long long)lineno);
            if (a < 0 || b < 0 || c < 0 || a >= (1ll << 31) || b >= (1ll << 31))
                return set_error(COMET_HIP_ERR_SIZE, "%s: dimensions %lld x %lld not supported", path, a, b);
            if (array && symmetric)
                return set_error(COMET_HIP_ERR_ARG, "%s: symmetric array files are not supported", path);
            out->nrows = a;
            out->ncols = b;
            declared = array ? a * b : (symmetric ? 2 * c : c);
            // every entry takes at least two bytes of text ("1\n" in an array file), so a count beyond the file's
            // size is a corrupt size line, not a reason to reserve memory for it
            if (declared > (int64_t)text.size() || declared >= (1ll << 32))
                return set_error(COMET_HIP_ERR_SIZE, "%s: the size line declares %lld entries, the file holds %lld bytes",
                                 path, (long long)declared, (long long)text.size());
            try {
                out->row.reserve((size_t)declared);
                out->col.reserve((size_t)declared);
                out->val.reserve((size_t)declared);
            } catch (const std::exception &) {
                return set_error(COMET_HIP_ERR_SIZE, "%s: no host memory for %lld entries", path, (long long)declared);
            }
            have_sizes = true;
            continue;
        }
        if (array) {
            const double v = strtod(l, &t);
            if (t == l)
                continue;
            if (array_seen >= declared)
                return set_error(COMET_HIP_ERR_ARG, "%s: more than %lld values", path, (long long)declared);
            out->row.push_back((int32_t)(array_seen % out->nrows));
            out->col.push_back((int32_t)(array_seen / out->nrows));
            out->val.push_back(v);
            ++array_seen;
            continue;
        }
        const long long r = strtoll(l, &t, 0);
        if (t == l)
            continue;          // blank line
        l = t;
        const long long c = strtoll(l, &t, 0);
        if (t == l)
            return set_error(COMET_HIP_ERR_ARG, "%s:%lld: badly formed column", path, (long long)lineno);
        l = t;
        double v = strtod(l, &t);
        if (t == l)
            v = 1.0;
        if (r < 1 || r > out->nrows || c < 1 || c > out->ncols)
            return set_error(COMET_HIP_ERR_ARG, "%s:%lld: entry (%lld,%lld) outside %lld x %lld", path,
                             (long long)lineno, r, c, (long long)out->nrows, (long long)out->ncols);
        if ((int64_t)out->row.size() + ((symmetric && r != c) ? 2 : 1) > declared)
            return set_error(COMET_HIP_ERR_ARG, "%s: more than the declared %lld entries", path,
                             (long long)declared);
        out->row.push_back((int32_t)(r - 1));
        out->col.push_back((int32_t)(c - 1));
        out->val.push_back(v);
        if (symmetric && r != c) {
            out->row.push_back((int32_t)(c - 1));
            out->col.push_back((int32_t)(r - 1));
            out->val.push_back(skew ? -v : v);
        }
    }
    if (!have_sizes)
        return set_error(COMET_HIP_ERR_ARG, "%s: no size line", path);
    return COMET_HIP_OK;
}

// ---------------------------------------------------------------------------
// Device tuples -> CSR.  key = row << 32 | col; a radix sort of (key, original
// position) is stable, so equal (row, col) pairs keep file order exactly as the
// reference's std::stable_sort does (SparseUtils.cpp:404-424; duplicates are
// kept, never merged).  Entries are then filtered by read mode (:458-507: 2
// strictly lower, 3 lower, 4 strictly upper, 5 upper, anything else all),
// compacted in order, and row r's pointer is the position of the first kept
// entry whose row is >= r.
// ---------------------------------------------------------------------------
// key = row << col_bits | col: no more bits than the matrix needs, because the radix sort's time goes with the
// number of key bits.  A tuple outside the matrix raises *bad (its key could not be told from another tuple's).
__global__ void coo_make_keys(int64_t n, const int32_t *__restrict__ row, const int32_t *__restrict__ col,
                              int64_t nrows, int64_t ncols, int col_bits, uint64_t *__restrict__ keys,
                              uint32_t *__restrict__ idx, int *__restrict__ bad)
{
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e < n) {
        const int64_t r = row[e], c = col[e];
        if (r < 0 || r >= nrows || c < 0 || c >= ncols) {
            atomicOr(bad, 1);
            keys[e] = 0;
        } else {
            keys[e] = ((uint64_t)r << col_bits) | (uint64_t)c;
        }
        idx[e] = (uint32_t)e;
    }
}

__device__ inline bool keep_entry(int mode, uint32_t r, uint32_t c)
{
    switch (mode) {
    case COMET_READ_LOWER_TRI_STRICT: return r > c;
    case COMET_READ_LOWER_TRI: return r >= c;
    case COMET_READ_UPPER_TRI_STRICT: return r < c;
    case COMET_READ_UPPER_TRI: return r <= c;
    default: return true;
    }
}

__global__ void coo_flag(int64_t n, const uint64_t *__restrict__ keys, int col_bits, int mode,
                         int64_t *__restrict__ flag)
{
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e < n)
        flag[e] = keep_entry(mode, (uint32_t)(keys[e] >> col_bits), (uint32_t)(keys[e] & ((1ull << col_bits) - 1))) ? 1 : 0;
}

__global__ void coo_compact(int64_t n, const uint64_t *__restrict__ keys, int col_bits,
                            const uint32_t *__restrict__ idx,
                            const int64_t *__restrict__ off, const double *__restrict__ val_in,
                            int32_t *__restrict__ crow, int32_t *__restrict__ crd, double *__restrict__ val)
{
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e < n && off[e + 1] != off[e]) {
        const int64_t o = off[e];
        crow[o] = (int32_t)(keys[e] >> col_bits);
        crd[o] = (int32_t)(keys[e] & ((1ull << col_bits) - 1));
        val[o] = val_in[idx[e]];
    }
}

// pos[r] = number of kept entries whose row is < r, for r in [0, nrows]
__global__ void rows_to_pos(int64_t nrows, int64_t kept, const int32_t *__restrict__ crow, int64_t *__restrict__ pos)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r > nrows)
        return;
    int64_t lo = 0, hi = kept;
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if (crow[mid] < r)
            lo = mid + 1;
        else
            hi = mid;
    }
    pos[r] = lo;
}

// rowid[e] = the row whose range [pos[r], pos[r+1]) holds entry e
__global__ void csr_expand_rows(int64_t nrows, int64_t nnz, const int64_t *__restrict__ pos,
                                int32_t *__restrict__ rowid)
{
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= nnz)
        return;
    int64_t lo = 0, hi = nrows;     // last r with pos[r] <= e
    while (lo < hi) {
        const int64_t mid = (lo + hi + 1) >> 1;
        if (pos[mid] <= e)
            lo = mid;
        else
            hi = mid - 1;
    }
    rowid[e] = (int32_t)lo;
}

// Kernels that give one lane to an entry read its row here instead of searching pos.
int csr_entry_rows(Csr *a, const int32_t **rows)
{
    if (!a->entry_row && a->nnz > 0) {
        if (a->nrows >= (1ll << 31))
            return set_error(COMET_HIP_ERR_SIZE, "row ids of %lld rows do not fit 32 bits", (long long)a->nrows);
        COMET_HIPCHK(hipMalloc((void **)&a->entry_row, sizeof(int32_t) * (size_t)a->nnz));
        KernelTimer t("csr_expand_rows");
        csr_expand_rows<<<dim3((unsigned)ceil_div(a->nnz, 256)), dim3(256), 0, stream()>>>(a->nrows, a->nnz, a->pos,
                                                                                           a->entry_row);
        COMET_HIPCHK(hipGetLastError());
    }
    *rows = a->entry_row;
    return COMET_HIP_OK;
}

__global__ void widen_i32(int64_t n, const int32_t *__restrict__ in, int64_t *__restrict__ out)
{
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e < n)
        out[e] = in[e];
}

// flag[r] = 1 if row r stores anything
__global__ void row_nonempty(int64_t nrows, const int64_t *__restrict__ pos, int64_t *__restrict__ flag)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r < nrows)
        flag[r] = pos[r + 1] != pos[r] ? 1 : 0;
}

__global__ void dcsr_compact_rows(int64_t nrows, const int64_t *__restrict__ pos, const int64_t *__restrict__ off,
                                  int64_t *__restrict__ a1crd, int64_t *__restrict__ a2pos)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r < nrows && off[r + 1] != off[r]) {
        a1crd[off[r]] = r;
        a2pos[off[r]] = pos[r];
    }
    if (r == nrows)
        a2pos[off[nrows]] = pos[nrows];
}

struct DevBuf {
    void *p = nullptr;
    ~DevBuf() { if (p) (void)hipFree(p); }
    int alloc(size_t bytes)
    {
        COMET_HIPCHK(hipMalloc(&p, bytes ? bytes : 1));
        return COMET_HIP_OK;
    }
    template <typename T> T *as() { return (T *)p; }
};

struct CachedBuf {
    Workspace w;
    void *p = nullptr;
    int alloc(size_t bytes)
    {
        COMET_CHK(w.ensure(bytes ? bytes : 1, false));
        p = w.ptr;
        return COMET_HIP_OK;
    }
    template <typename T> T *as() { return (T *)p; }
};

int sort_pairs_u64_u32(const uint64_t *keys_in, uint64_t *keys_out, const uint32_t *vals_in, uint32_t *vals_out,
                       int64_t n, int end_bit)
{
    static Workspace tmp;
    if (n <= 0)
        return COMET_HIP_OK;
    size_t tmp_bytes = 0;
    if (rocprim::radix_sort_pairs(nullptr, tmp_bytes, keys_in, keys_out, vals_in, vals_out, (size_t)n, 0u,
                                  (unsigned)end_bit, stream()) != hipSuccess)
        return set_error(COMET_HIP_ERR_HIP, "sort workspace query failed");
    COMET_CHK(tmp.ensure(tmp_bytes ? tmp_bytes : 1, false));
    KernelTimer t("radix_sort_pairs");
    if (rocprim::radix_sort_pairs(tmp.ptr, tmp_bytes, keys_in, keys_out, vals_in, vals_out, (size_t)n, 0u,
                                  (unsigned)end_bit, stream()) != hipSuccess)
        return set_error(COMET_HIP_ERR_HIP, "sorting %lld pairs failed", (long long)n);
    return COMET_HIP_OK;
}

static inline dim3 grid_for(int64_t n) { return dim3((unsigned)(n > 0 ? ceil_div(n, 256) : 1)); }

// row/col/val are device arrays of n tuples in input order; returns a new registered handle or 0
static Csr *coo_device_to_csr_struct(int64_t nrows, int64_t ncols, int64_t n, const int32_t *row,
                                     const int32_t *col, const double *val, int mode);

static int64_t coo_device_to_csr(int64_t nrows, int64_t ncols, int64_t n, const int32_t *row, const int32_t *col,
                                 const double *val, int mode)
{
    Csr *c = coo_device_to_csr_struct(nrows, ncols, n, row, col, val, mode);
    return c ? csr_register(c) : 0;
}

// the same, as a struct that no handle names yet (nullptr on failure)
static Csr *coo_device_to_csr_struct(int64_t nrows, int64_t ncols, int64_t n, const int32_t *row,
                                     const int32_t *col, const double *val, int mode)
{
    Csr *c = new Csr();
    c->nrows = nrows;
    c->ncols = ncols;
    c->owns = true;
    auto fail = [&]() -> Csr * {
        (void)hipFree(c->pos);
        (void)hipFree(c->crd);
        (void)hipFree(c->val);
        delete c;
        return nullptr;
    };
    if (hipMalloc((void **)&c->pos, sizeof(int64_t) * (size_t)(nrows + 1)) != hipSuccess) {
        set_error(COMET_HIP_ERR_HIP, "row pointer allocation failed");
        return fail();
    }
    // temporaries live in grow-only buffers kept for the life of the process: a conversion of a few million
    // tuples takes less time than the allocations would
    static CachedBuf keys_in, keys_out, idx_in, idx_out, flag, off, crow, bad;
    int64_t kept = 0;
    int row_bits = 1, col_bits = 1;
    while (row_bits < 31 && (1ll << row_bits) < nrows)
        ++row_bits;
    while (col_bits < 31 && (1ll << col_bits) < ncols)
        ++col_bits;
    if (n > 0) {
        if (keys_in.alloc(8 * (size_t)n) || keys_out.alloc(8 * (size_t)n) || idx_in.alloc(4 * (size_t)n) ||
            idx_out.alloc(4 * (size_t)n) || flag.alloc(8 * (size_t)n) || off.alloc(8 * (size_t)(n + 1)) ||
            bad.alloc(sizeof(int)))
            return fail();
        if (hipMemsetAsync(bad.p, 0, sizeof(int), stream()) != hipSuccess) {
            set_error(COMET_HIP_ERR_HIP, "clearing the range flag failed");
            return fail();
        }
        {
            KernelTimer t("coo_make_keys");
            coo_make_keys<<<grid_for(n), dim3(256), 0, stream()>>>(n, row, col, nrows, ncols, col_bits,
                                                                  keys_in.as<uint64_t>(), idx_in.as<uint32_t>(),
                                                                  bad.as<int>());
        }
        if (sort_pairs_u64_u32(keys_in.as<uint64_t>(), keys_out.as<uint64_t>(), idx_in.as<uint32_t>(),
                               idx_out.as<uint32_t>(), n, col_bits + row_bits) != COMET_HIP_OK)
            return fail();
        {
            KernelTimer t("coo_flag");
            coo_flag<<<grid_for(n), dim3(256), 0, stream()>>>(n, keys_out.as<uint64_t>(), col_bits, mode,
                                                             flag.as<int64_t>());
        }
        if (exclusive_scan_i64(flag.as<int64_t>(), n, off.as<int64_t>()) != COMET_HIP_OK)
            return fail();
        int any_bad = 0;
        if (hipMemcpyAsync(&kept, off.as<int64_t>() + n, sizeof(int64_t), hipMemcpyDeviceToHost, stream()) !=
                hipSuccess ||
            hipMemcpyAsync(&any_bad, bad.p, sizeof(int), hipMemcpyDeviceToHost, stream()) != hipSuccess ||
            hipStreamSynchronize(stream()) != hipSuccess) {
            set_error(COMET_HIP_ERR_HIP, "reading the entry count failed");
            return fail();
        }
        if (any_bad) {
            set_error(COMET_HIP_ERR_ARG, "a tuple lies outside the %lld x %lld matrix", (long long)nrows,
                      (long long)ncols);
            return fail();
        }
    }
    c->nnz = kept;
    if (hipMalloc((void **)&c->crd, sizeof(int32_t) * (size_t)(kept > 0 ? kept : 1)) != hipSuccess ||
        hipMalloc((void **)&c->val, sizeof(double) * (size_t)(kept > 0 ? kept : 1)) != hipSuccess ||
        crow.alloc(4 * (size_t)(kept > 0 ? kept : 1))) {
        set_error(COMET_HIP_ERR_HIP, "allocation of %lld entries failed", (long long)kept);
        return fail();
    }
    if (n > 0) {
        KernelTimer t("coo_compact");
        coo_compact<<<grid_for(n), dim3(256), 0, stream()>>>(n, keys_out.as<uint64_t>(), col_bits,
                                                            idx_out.as<uint32_t>(),
                                                            off.as<int64_t>(), val, crow.as<int32_t>(), c->crd,
                                                            c->val);
    }
    {
        KernelTimer t("rows_to_pos");
        rows_to_pos<<<grid_for(nrows + 1), dim3(256), 0, stream()>>>(nrows, kept, crow.as<int32_t>(), c->pos);
    }
    if (hipGetLastError() != hipSuccess || hipStreamSynchronize(stream()) != hipSuccess) {
        set_error(COMET_HIP_ERR_HIP, "building the CSR arrays failed");
        return fail();
    }
    return c;
}

static int64_t coo_host_to_csr(int64_t nrows, int64_t ncols, int64_t n, const int32_t *row, const int32_t *col,
                               const double *val, int mode)
{
    DevBuf drow, dcol, dval;
    if (drow.alloc(4 * (size_t)n) || dcol.alloc(4 * (size_t)n) || dval.alloc(8 * (size_t)n))
        return 0;
    if (n > 0 &&
        (hipMemcpyAsync(drow.p, row, 4 * (size_t)n, hipMemcpyHostToDevice, stream()) != hipSuccess ||
         hipMemcpyAsync(dcol.p, col, 4 * (size_t)n, hipMemcpyHostToDevice, stream()) != hipSuccess ||
         hipMemcpyAsync(dval.p, val, 8 * (size_t)n, hipMemcpyHostToDevice, stream()) != hipSuccess ||
         hipStreamSynchronize(stream()) != hipSuccess)) {
        set_error(COMET_HIP_ERR_HIP, "uploading %lld tuples failed", (long long)n);
        return 0;
    }
    return coo_device_to_csr(nrows, ncols, n, drow.as<int32_t>(), dcol.as<int32_t>(), dval.as<double>(), mode);
}

Csr *csr_transposed_copy(const Csr *a)
{
    DevBuf rowid;
    if (rowid.alloc(4 * (size_t)a->nnz))
        return nullptr;
    if (a->nnz > 0) {
        KernelTimer t("csr_expand_rows");
        csr_expand_rows<<<grid_for(a->nnz), dim3(256), 0, stream()>>>(a->nrows, a->nnz, a->pos, rowid.as<int32_t>());
    }
    // the tuples of the transpose are (column, row, value): order them by (column, row)
    return coo_device_to_csr_struct(a->ncols, a->nrows, a->nnz, a->crd, rowid.as<int32_t>(), a->val,
                                    COMET_READ_DEFAULT);
}

static bool known_mode(int mode) { return mode >= COMET_READ_DEFAULT && mode <= COMET_READ_UPPER_TRI; }

// ---------------------------------------------------------------------------
// The reader's file-id protocol (SparseUtils.cpp:1425-1600): id 0..9998 names
// the environment variable SPARSE_FILE_NAME<id>, 9999 plain SPARSE_FILE_NAME.
// The sizes call reads the file and keeps the result; the read call that
// follows consumes it.  What is kept here is the finished device CSR.
// ---------------------------------------------------------------------------
static std::map<std::pair<int32_t, int32_t>, int64_t> g_pending_reads;

void comet::forget_pending_reads() { g_pending_reads.clear(); }

static int file_name_of(int32_t file_id, std::string *out)
{
    const char *v = nullptr;
    if (file_id >= 0 && file_id < 9999)
        v = getenv(("SPARSE_FILE_NAME" + std::to_string(file_id)).c_str());
    else if (file_id == 9999)
        v = getenv("SPARSE_FILE_NAME");
    if (!v || !*v)
        return set_error(COMET_HIP_ERR_ARG, "SPARSE_FILE_NAME%s is not set",
                         file_id == 9999 ? "" : std::to_string(file_id).c_str());
    *out = v;
    if (out->find(".mtx") == std::string::npos)
        return set_error(COMET_HIP_ERR_ARG, "%s is not a Matrix Market file", v);
    return COMET_HIP_OK;
}

static int64_t pending_read(int32_t file_id, int32_t mode, bool take)
{
    const int32_t m = known_mode(mode) ? mode : COMET_READ_DEFAULT;   // getMatrixReadOption, SparseUtils.cpp:50-64
    auto key = std::make_pair(file_id, m);
    auto it = g_pending_reads.find(key);
    int64_t h = 0;
    if (it != g_pending_reads.end()) {
        h = it->second;
    } else {
        std::string name;
        if (file_name_of(file_id, &name) != COMET_HIP_OK)
            return 0;
        h = comet_hip_mtx_read_csr(name.c_str(), m);
        if (!h)
            return 0;
        g_pending_reads[key] = h;
    }
    if (take)
        g_pending_reads.erase(key);
    return h;
}

static void die_reader(const char *who)
{
    fprintf(stderr, "%s: %s\n", who, comet_hip_last_error());
    exit(1);
}

enum Layout { LAYOUT_CSR, LAYOUT_COO, LAYOUT_DCSR, LAYOUT_OTHER };
static Layout layout_of(int32_t a1, int32_t a1_tile, int32_t a2, int32_t a2_tile)
{
    (void)a2_tile;
    if (a1 == COMET_FMT_COMPRESSED_NONUNIQUE && a2 == COMET_FMT_SINGLETON)
        return LAYOUT_COO;
    if (a1 == COMET_FMT_DENSE && a2 == COMET_FMT_COMPRESSED_UNIQUE)
        return LAYOUT_CSR;
    if (a1 == COMET_FMT_COMPRESSED_UNIQUE && a2 == COMET_FMT_COMPRESSED_UNIQUE)
        return LAYOUT_DCSR;
    (void)a1_tile;
    return LAYOUT_OTHER;
}

template <typename T>
static T *memref_data(void *desc)
{
    auto *m = (comet_memref_1d *)desc;
    return m && m->aligned ? (T *)m->aligned + m->offset : nullptr;
}

}  // namespace comet

using namespace comet;

extern "C" int64_t comet_hip_mtx_read_csr(const char *path, int read_mode)
{
    if (ensure_init() != COMET_HIP_OK)
        return 0;
    if (!path) {
        set_error(COMET_HIP_ERR_ARG, "null path passed to comet_hip_mtx_read_csr");
        return 0;
    }
    if (!known_mode(read_mode)) {
        set_error(COMET_HIP_ERR_ARG, "unknown read mode %d", read_mode);
        return 0;
    }
    HostCoo coo;
    if (parse_mtx(path, &coo) != COMET_HIP_OK)
        return 0;
    return coo_host_to_csr(coo.nrows, coo.ncols, (int64_t)coo.row.size(), coo.row.data(), coo.col.data(),
                           coo.val.data(), read_mode);
}

extern "C" int64_t comet_hip_csr_from_coo_i64(int64_t nrows, int64_t ncols, int64_t nnz, const int64_t *row,
                                              const int64_t *col, const double *val, int read_mode)
{
    if (ensure_init() != COMET_HIP_OK)
        return 0;
    if (nrows < 0 || ncols < 0 || nnz < 0 || nrows >= (1ll << 31) || ncols >= (1ll << 31) || nnz >= (1ll << 32) ||
        (nnz > 0 && (!row || !col || !val)) || !known_mode(read_mode)) {
        set_error(COMET_HIP_ERR_ARG, "bad arguments to comet_hip_csr_from_coo_i64 (%lld x %lld, %lld entries, mode %d)",
                  (long long)nrows, (long long)ncols, (long long)nnz, read_mode);
        return 0;
    }
    std::vector<int32_t> r32, c32;
    try {
        r32.resize((size_t)nnz);
        c32.resize((size_t)nnz);
    } catch (const std::exception &) {
        set_error(COMET_HIP_ERR_SIZE, "no host memory to stage %lld tuples", (long long)nnz);
        return 0;
    }
    for (int64_t e = 0; e < nnz; ++e) {
        if (row[e] < 0 || row[e] >= nrows || col[e] < 0 || col[e] >= ncols) {
            set_error(COMET_HIP_ERR_ARG, "tuple %lld = (%lld,%lld) lies outside %lld x %lld", (long long)e,
                      (long long)row[e], (long long)col[e], (long long)nrows, (long long)ncols);
            return 0;
        }
        r32[(size_t)e] = (int32_t)row[e];
        c32[(size_t)e] = (int32_t)col[e];
    }
    return coo_host_to_csr(nrows, ncols, nnz, r32.data(), c32.data(), val, read_mode);
}

extern "C" int64_t comet_hip_csr_from_coo_device(int64_t nrows, int64_t ncols, int64_t nnz, int64_t row_dptr,
                                                 int64_t col_dptr, int64_t val_dptr, int read_mode)
{
    if (ensure_init() != COMET_HIP_OK)
        return 0;
    if (nrows < 0 || ncols < 0 || nnz < 0 || nrows >= (1ll << 31) || ncols >= (1ll << 31) || nnz >= (1ll << 32) ||
        (nnz > 0 && (!row_dptr || !col_dptr || !val_dptr)) || !known_mode(read_mode)) {
        set_error(COMET_HIP_ERR_ARG, "bad arguments to comet_hip_csr_from_coo_device (%lld x %lld, %lld entries, mode %d)",
                  (long long)nrows, (long long)ncols, (long long)nnz, read_mode);
        return 0;
    }
    return coo_device_to_csr(nrows, ncols, nnz, (const int32_t *)row_dptr, (const int32_t *)col_dptr,
                             (const double *)val_dptr, read_mode);
}

extern "C" int64_t comet_hip_csr_from_dcsr_i64(int64_t nrows, int64_t ncols, int64_t nrows_stored,
                                               const int64_t *a1crd, const int64_t *a2pos, const int64_t *a2crd,
                                               const double *aval)
{
    if (ensure_init() != COMET_HIP_OK)
        return 0;
    if (nrows < 0 || nrows_stored < 0 || nrows_stored > nrows || !a2pos || (nrows_stored > 0 && !a1crd)) {
        set_error(COMET_HIP_ERR_ARG, "bad arguments to comet_hip_csr_from_dcsr_i64");
        return 0;
    }
    // expand the stored-row list into one pointer per row; the arrays of the second level are CSR's already
    std::vector<int64_t> pos;
    try {
        pos.assign((size_t)nrows + 1, 0);
    } catch (const std::exception &) {
        set_error(COMET_HIP_ERR_SIZE, "no host memory for the row pointers of %lld rows", (long long)nrows);
        return 0;
    }
    int64_t prev = -1;
    for (int64_t s = 0; s < nrows_stored; ++s) {
        const int64_t r = a1crd[s];
        if (r <= prev || r >= nrows || a2pos[s + 1] < a2pos[s]) {
            set_error(COMET_HIP_ERR_ARG, "stored row %lld (row id %lld) is out of order or out of range",
                      (long long)s, (long long)r);
            return 0;
        }
        for (int64_t q = prev + 1; q <= r; ++q)
            pos[(size_t)q] = a2pos[s];
        prev = r;
    }
    for (int64_t q = prev + 1; q <= nrows; ++q)
        pos[(size_t)q] = a2pos[nrows_stored];
    if (pos[0] != 0) {
        set_error(COMET_HIP_ERR_ARG, "the second-level pointers must start at 0");
        return 0;
    }
    return comet_hip_csr_upload_i64(nrows, ncols, pos.data(), a2crd, aval);
}

extern "C" int comet_hip_csr_to_coo_i64(int64_t h, int64_t *row, int64_t *col, double *val)
{
    COMET_CHK(ensure_init());
    Csr *a = csr_from_handle(h);
    if (!a)
        return COMET_HIP_ERR_HANDLE;
    if (a->nnz == 0)
        return COMET_HIP_OK;
    if (!row || !col || !val)
        return set_error(COMET_HIP_ERR_ARG, "null output passed to comet_hip_csr_to_coo_i64");
    DevBuf r32, wide;
    COMET_CHK(r32.alloc(4 * (size_t)a->nnz));
    COMET_CHK(wide.alloc(8 * (size_t)a->nnz));
    {
        KernelTimer t("csr_expand_rows");
        csr_expand_rows<<<grid_for(a->nnz), dim3(256), 0, stream()>>>(a->nrows, a->nnz, a->pos, r32.as<int32_t>());
    }
    widen_i32<<<grid_for(a->nnz), dim3(256), 0, stream()>>>(a->nnz, r32.as<int32_t>(), wide.as<int64_t>());
    COMET_HIPCHK(hipMemcpyAsync(row, wide.p, 8 * (size_t)a->nnz, hipMemcpyDeviceToHost, stream()));
    widen_i32<<<grid_for(a->nnz), dim3(256), 0, stream()>>>(a->nnz, a->crd, wide.as<int64_t>());
    COMET_HIPCHK(hipMemcpyAsync(col, wide.p, 8 * (size_t)a->nnz, hipMemcpyDeviceToHost, stream()));
    COMET_HIPCHK(hipMemcpyAsync(val, a->val, 8 * (size_t)a->nnz, hipMemcpyDeviceToHost, stream()));
    COMET_HIPCHK(hipStreamSynchronize(stream()));
    return COMET_HIP_OK;
}

extern "C" int comet_hip_csr_to_dcsr_i64(int64_t h, int64_t *nrows_stored, int64_t *a1crd, int64_t *a2pos,
                                         int64_t *a2crd, double *aval)
{
    COMET_CHK(ensure_init());
    Csr *a = csr_from_handle(h);
    if (!a)
        return COMET_HIP_ERR_HANDLE;
    if (!nrows_stored)
        return set_error(COMET_HIP_ERR_ARG, "null count passed to comet_hip_csr_to_dcsr_i64");
    DevBuf flag, off, d1, d2, wide;
    COMET_CHK(flag.alloc(8 * (size_t)(a->nrows + 1)));
    COMET_CHK(off.alloc(8 * (size_t)(a->nrows + 1)));
    int64_t stored = 0;
    if (a->nrows > 0) {
        row_nonempty<<<grid_for(a->nrows), dim3(256), 0, stream()>>>(a->nrows, a->pos, flag.as<int64_t>());
        COMET_CHK(exclusive_scan_i64(flag.as<int64_t>(), a->nrows, off.as<int64_t>()));
        COMET_HIPCHK(hipMemcpyAsync(&stored, off.as<int64_t>() + a->nrows, 8, hipMemcpyDeviceToHost, stream()));
        COMET_HIPCHK(hipStreamSynchronize(stream()));
    }
    *nrows_stored = stored;
    if (!a1crd && !a2pos && !a2crd && !aval)
        return COMET_HIP_OK;            // size query
    if (!a1crd || !a2pos || (a->nnz > 0 && (!a2crd || !aval)))
        return set_error(COMET_HIP_ERR_ARG, "null output passed to comet_hip_csr_to_dcsr_i64");
    if (a->nrows == 0) {
        a2pos[0] = 0;
        return COMET_HIP_OK;
    }
    COMET_CHK(d1.alloc(8 * (size_t)stored));
    COMET_CHK(d2.alloc(8 * (size_t)(stored + 1)));
    {
        KernelTimer t("dcsr_compact_rows");
        dcsr_compact_rows<<<grid_for(a->nrows + 1), dim3(256), 0, stream()>>>(a->nrows, a->pos, off.as<int64_t>(),
                                                                             d1.as<int64_t>(), d2.as<int64_t>());
    }
    COMET_HIPCHK(hipMemcpyAsync(a1crd, d1.p, 8 * (size_t)stored, hipMemcpyDeviceToHost, stream()));
    COMET_HIPCHK(hipMemcpyAsync(a2pos, d2.p, 8 * (size_t)(stored + 1), hipMemcpyDeviceToHost, stream()));
    if (a->nnz > 0) {
        COMET_CHK(wide.alloc(8 * (size_t)a->nnz));
        widen_i32<<<grid_for(a->nnz), dim3(256), 0, stream()>>>(a->nnz, a->crd, wide.as<int64_t>());
        COMET_HIPCHK(hipMemcpyAsync(a2crd, wide.p, 8 * (size_t)a->nnz, hipMemcpyDeviceToHost, stream()));
        COMET_HIPCHK(hipMemcpyAsync(aval, a->val, 8 * (size_t)a->nnz, hipMemcpyDeviceToHost, stream()));
    }
    COMET_HIPCHK(hipStreamSynchronize(stream()));
    return COMET_HIP_OK;
}

extern "C" int64_t comet_hip_csr_transpose(int64_t h)
{
    if (ensure_init() != COMET_HIP_OK)
        return 0;
    Csr *a = csr_from_handle(h);
    if (!a)
        return 0;
    Csr *t = csr_transposed_copy(a);
    return t ? csr_register(t) : 0;
}

extern "C" int64_t comet_hip_read_input_2D_handle(int32_t file_id, int32_t read_mode)
{
    if (ensure_init() != COMET_HIP_OK)
        return 0;
    return pending_read(file_id, read_mode, true);
}

extern "C" void comet_hip_read_input_sizes_2D_f64(int32_t file_id, int32_t a1format, int32_t a1_tile_format,
                                                  int32_t a2format, int32_t a2_tile_format, int sizes_rank,
                                                  void *sizes_desc, int32_t read_mode)
{
    const char *who = "comet_hip_read_input_sizes_2D_f64";
    (void)sizes_rank;
    int64_t *s = memref_data<int64_t>(sizes_desc);
    const Layout lay = layout_of(a1format, a1_tile_format, a2format, a2_tile_format);
    if (!s || lay == LAYOUT_OTHER) {
        set_error(COMET_HIP_ERR_ARG, "only CSR, COO and DCSR layouts are read (formats %d,%d)", a1format, a2format);
        die_reader(who);
    }
    if (ensure_init() != COMET_HIP_OK)
        die_reader(who);
    const int64_t h = pending_read(file_id, read_mode, false);
    if (!h)
        die_reader(who);
    int64_t nrows = 0, ncols = 0, nnz = 0;
    (void)comet_hip_csr_dims(h, &nrows, &ncols, &nnz);
    for (int i = 0; i < 8; ++i)
        s[i] = 0;
    if (lay == LAYOUT_COO) {            // SparseUtils.cpp:1643-1659
        s[0] = 2;
        s[1] = nnz;
        s[4] = 1;
        s[5] = nnz;
    } else if (lay == LAYOUT_CSR) {     // :1672-1687
        s[0] = 1;
        s[1] = 1;
        s[4] = nrows + 1;
        s[5] = nnz;
    } else {                            // DCSR, :1731-1749 with the array sizes of :669-735
        int64_t stored = 0;
        if (comet_hip_csr_to_dcsr_i64(h, &stored, nullptr, nullptr, nullptr, nullptr))
            die_reader(who);
        s[0] = 2;
        s[1] = stored;
        s[4] = stored + 1;
        s[5] = nnz;
    }
    s[8] = nnz;
    s[9] = nrows;
    s[10] = ncols;
}

// I = int64_t for the CPU lowering, int32_t for lowered code built with --target=GPU, which switches every index
// memref to i32 (frontends/comet_dsl/comet.cpp:817-823); the reference's reader is one template over both
// (SparseUtils.cpp:2403-2447).
template <typename I>
static void read_input_2D_impl(const char *who, int32_t file_id, int32_t a1format, int32_t a1_tile_format,
                               int32_t a2format, int32_t a2_tile_format, void *a1pos_desc, void *a1crd_desc,
                               void *a1tile_pos_desc, void *a1tile_crd_desc, void *a2pos_desc, void *a2crd_desc,
                               void *a2tile_pos_desc, void *a2tile_crd_desc, void *aval_desc, int32_t read_mode)
{
    I *a1pos = memref_data<I>(a1pos_desc), *a1crd = memref_data<I>(a1crd_desc);
    I *a2pos = memref_data<I>(a2pos_desc), *a2crd = memref_data<I>(a2crd_desc);
    double *aval = memref_data<double>(aval_desc);
    const Layout lay = layout_of(a1format, a1_tile_format, a2format, a2_tile_format);
    if (lay == LAYOUT_OTHER || !a1pos || !a1crd || !a2pos || !a2crd || !aval) {
        set_error(COMET_HIP_ERR_ARG, "only CSR, COO and DCSR layouts are read (formats %d,%d), all arrays required",
                  a1format, a2format);
        die_reader(who);
    }
    if (ensure_init() != COMET_HIP_OK)
        die_reader(who);
    // arrays a layout does not use hold -1 in their first element (SparseUtils.cpp:1840-1848)
    void *all[8] = {a1pos_desc, a1crd_desc, a2pos_desc, a2crd_desc,
                    a1tile_pos_desc, a1tile_crd_desc, a2tile_pos_desc, a2tile_crd_desc};
    for (void *d : all) {
        I *p = memref_data<I>(d);
        if (p && ((comet_memref_1d *)d)->sizes[0] > 0)
            p[0] = -1;
    }
    const int64_t h = pending_read(file_id, read_mode, true);
    if (!h)
        die_reader(who);
    int64_t nrows = 0, nnz = 0;
    (void)comet_hip_csr_dims(h, &nrows, nullptr, &nnz);
    int rc = COMET_HIP_OK;
    if constexpr (sizeof(I) == 8) {
        int64_t *p1 = (int64_t *)a1pos, *c1 = (int64_t *)a1crd, *p2 = (int64_t *)a2pos, *c2 = (int64_t *)a2crd;
        if (lay == LAYOUT_CSR) {            // :1898-1936
            p1[0] = nrows;
            rc = comet_hip_csr_download_i64(h, p2, c2, aval);
        } else if (lay == LAYOUT_COO) {     // :1855-1896
            p1[0] = 0;
            p1[1] = nnz;
            rc = comet_hip_csr_to_coo_i64(h, c1, c2, aval);
        } else {                            // DCSR :1983-2010
            int64_t stored = 0;
            rc = comet_hip_csr_to_dcsr_i64(h, &stored, c1, p2, c2, aval);
            p1[0] = 0;
            p1[1] = stored;
        }
    } else {
        int32_t *p1 = (int32_t *)a1pos, *c1 = (int32_t *)a1crd, *p2 = (int32_t *)a2pos, *c2 = (int32_t *)a2crd;
        if (nnz > INT32_MAX) {
            set_error(COMET_HIP_ERR_SIZE, "%lld entries do not fit 32-bit positions", (long long)nnz);
            rc = COMET_HIP_ERR_SIZE;
        } else if (lay == LAYOUT_CSR) {
            p1[0] = (int32_t)nrows;
            rc = comet_hip_csr_download_i32(h, p2, c2, aval);
        } else {
            // the COO and DCSR conversions produce 64-bit host arrays: narrow them here
            std::vector<int64_t> w1, w2, wp;
            try {
                w1.resize((size_t)std::max<int64_t>(lay == LAYOUT_COO ? nnz : nrows, 1));
                w2.resize((size_t)std::max<int64_t>(nnz, 1));
                wp.resize((size_t)nrows + 1);
            } catch (const std::exception &) {
                set_error(COMET_HIP_ERR_SIZE, "no host memory to stage %lld entries", (long long)nnz);
                die_reader(who);
            }
            if (lay == LAYOUT_COO) {
                p1[0] = 0;
                p1[1] = (int32_t)nnz;
                rc = comet_hip_csr_to_coo_i64(h, w1.data(), w2.data(), aval);
                for (int64_t e = 0; rc == COMET_HIP_OK && e < nnz; ++e) {
                    c1[e] = (int32_t)w1[(size_t)e];
                    c2[e] = (int32_t)w2[(size_t)e];
                }
            } else {
                int64_t stored = 0;
                rc = comet_hip_csr_to_dcsr_i64(h, &stored, w1.data(), wp.data(), w2.data(), aval);
                p1[0] = 0;
                p1[1] = (int32_t)stored;
                for (int64_t r = 0; rc == COMET_HIP_OK && r < stored; ++r)
                    c1[r] = (int32_t)w1[(size_t)r];
                for (int64_t r = 0; rc == COMET_HIP_OK && r <= stored; ++r)
                    p2[r] = (int32_t)wp[(size_t)r];
                for (int64_t e = 0; rc == COMET_HIP_OK && e < nnz; ++e)
                    c2[e] = (int32_t)w2[(size_t)e];
            }
        }
    }
    (void)comet_hip_csr_destroy(h);
    if (rc)
        die_reader(who);
}

extern "C" void comet_hip_read_input_2D_f64_i64(int32_t file_id, int32_t a1format, int32_t a1_tile_format,
                                                int32_t a2format, int32_t a2_tile_format, int a1pos_rank,
                                                void *a1pos_desc, int a1crd_rank, void *a1crd_desc,
                                                int a1tile_pos_rank, void *a1tile_pos_desc, int a1tile_crd_rank,
                                                void *a1tile_crd_desc, int a2pos_rank, void *a2pos_desc,
                                                int a2crd_rank, void *a2crd_desc, int a2tile_pos_rank,
                                                void *a2tile_pos_desc, int a2tile_crd_rank, void *a2tile_crd_desc,
                                                int aval_rank, void *aval_desc, int32_t read_mode)
{
    (void)a1pos_rank; (void)a1crd_rank; (void)a1tile_pos_rank; (void)a1tile_crd_rank; (void)a2pos_rank;
    (void)a2crd_rank; (void)a2tile_pos_rank; (void)a2tile_crd_rank; (void)aval_rank;
    read_input_2D_impl<int64_t>("comet_hip_read_input_2D_f64_i64", file_id, a1format, a1_tile_format, a2format,
                                a2_tile_format, a1pos_desc, a1crd_desc, a1tile_pos_desc, a1tile_crd_desc, a2pos_desc,
                                a2crd_desc, a2tile_pos_desc, a2tile_crd_desc, aval_desc, read_mode);
}

extern "C" void comet_hip_read_input_2D_f64_i32(int32_t file_id, int32_t a1format, int32_t a1_tile_format,
                                                int32_t a2format, int32_t a2_tile_format, int a1pos_rank,
                                                void *a1pos_desc, int a1crd_rank, void *a1crd_desc,
                                                int a1tile_pos_rank, void *a1tile_pos_desc, int a1tile_crd_rank,
                                                void *a1tile_crd_desc, int a2pos_rank, void *a2pos_desc,
                                                int a2crd_rank, void *a2crd_desc, int a2tile_pos_rank,
                                                void *a2tile_pos_desc, int a2tile_crd_rank, void *a2tile_crd_desc,
                                                int aval_rank, void *aval_desc, int32_t read_mode)
{
    (void)a1pos_rank; (void)a1crd_rank; (void)a1tile_pos_rank; (void)a1tile_crd_rank; (void)a2pos_rank;
    (void)a2crd_rank; (void)a2tile_pos_rank; (void)a2tile_crd_rank; (void)aval_rank;
    read_input_2D_impl<int32_t>("comet_hip_read_input_2D_f64_i32", file_id, a1format, a1_tile_format, a2format,
                                a2_tile_format, a1pos_desc, a1crd_desc, a1tile_pos_desc, a1tile_crd_desc, a2pos_desc,
                                a2crd_desc, a2tile_pos_desc, a2tile_crd_desc, aval_desc, read_mode);
}

// The reader under the names lowered code calls (lib/ExecutionEngine/SparseUtils.cpp:2403-2450, 2562-2568): with
// this library in -shared-libs in place of libcomet_runner_utils, `ta.read` resolves without a compiler change.
// Same argument lists, same behaviour as the comet_hip_read_input_* functions above.
extern "C" void read_input_sizes_2D_f64(int32_t file_id, int32_t a1format, int32_t a1_tile_format, int32_t a2format,
                                        int32_t a2_tile_format, int sizes_rank, void *sizes_desc, int32_t read_mode)
{
    comet_hip_read_input_sizes_2D_f64(file_id, a1format, a1_tile_format, a2format, a2_tile_format, sizes_rank,
                                      sizes_desc, read_mode);
}

extern "C" void read_input_2D_f64_i64(int32_t file_id, int32_t a1format, int32_t a1_tile_format, int32_t a2format,
                                      int32_t a2_tile_format, int a1pos_rank, void *a1pos_desc, int a1crd_rank,
                                      void *a1crd_desc, int a1tile_pos_rank, void *a1tile_pos_desc, int a1tile_crd_rank,
                                      void *a1tile_crd_desc, int a2pos_rank, void *a2pos_desc, int a2crd_rank,
                                      void *a2crd_desc, int a2tile_pos_rank, void *a2tile_pos_desc, int a2tile_crd_rank,
                                      void *a2tile_crd_desc, int aval_rank, void *aval_desc, int32_t read_mode)
{
    comet_hip_read_input_2D_f64_i64(file_id, a1format, a1_tile_format, a2format, a2_tile_format, a1pos_rank, a1pos_desc,
                                    a1crd_rank, a1crd_desc, a1tile_pos_rank, a1tile_pos_desc, a1tile_crd_rank,
                                    a1tile_crd_desc, a2pos_rank, a2pos_desc, a2crd_rank, a2crd_desc, a2tile_pos_rank,
                                    a2tile_pos_desc, a2tile_crd_rank, a2tile_crd_desc, aval_rank, aval_desc, read_mode);
}

extern "C" void read_input_2D_f64_i32(int32_t file_id, int32_t a1format, int32_t a1_tile_format, int32_t a2format,
                                      int32_t a2_tile_format, int a1pos_rank, void *a1pos_desc, int a1crd_rank,
                                      void *a1crd_desc, int a1tile_pos_rank, void *a1tile_pos_desc, int a1tile_crd_rank,
                                      void *a1tile_crd_desc, int a2pos_rank, void *a2pos_desc, int a2crd_rank,
                                      void *a2crd_desc, int a2tile_pos_rank, void *a2tile_pos_desc, int a2tile_crd_rank,
                                      void *a2tile_crd_desc, int aval_rank, void *aval_desc, int32_t read_mode)
{
    comet_hip_read_input_2D_f64_i32(file_id, a1format, a1_tile_format, a2format, a2_tile_format, a1pos_rank, a1pos_desc,
                                    a1crd_rank, a1crd_desc, a1tile_pos_rank, a1tile_pos_desc, a1tile_crd_rank,
                                    a1tile_crd_desc, a2pos_rank, a2pos_desc, a2crd_rank, a2crd_desc, a2tile_pos_rank,
                                    a2tile_pos_desc, a2tile_crd_rank, a2tile_crd_desc, aval_rank, aval_desc, read_mode);
}
