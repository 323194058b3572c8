// Device runtime: lifetime, errors, raw memory, CSR handles, scan, reduction,
// event timing.  Takes the place of the reference's Hip* host glue
// (lib/ExecutionEngine/HipGpuUtils.cpp in pnnl/COMET) and of the host-side
// tensor utilities the lowered code used around its loop nests.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <map>
#include <atomic>
#include <mutex>
#include <unordered_set>

#include "common.h"

namespace comet {

static std::mutex g_mu;
static bool g_inited = false;
static int g_device = 0;
static int g_num_cus = 0;
static hipStream_t g_stream = nullptr;
static hipStream_t g_aux = nullptr;
static hipEvent_t g_fork = nullptr, g_join = nullptr;
static thread_local std::string g_last_error;
static std::unordered_set<Csr *> g_live;

hipStream_t stream() { return g_stream; }
hipStream_t aux_stream() { return g_aux; }

int aux_fork()
{
    COMET_HIPCHK(hipEventRecord(g_fork, g_stream));
    COMET_HIPCHK(hipStreamWaitEvent(g_aux, g_fork, 0));
    return COMET_HIP_OK;
}

int aux_join()
{
    COMET_HIPCHK(hipEventRecord(g_join, g_aux));
    COMET_HIPCHK(hipStreamWaitEvent(g_stream, g_join, 0));
    return COMET_HIP_OK;
}
int num_cus() { return g_num_cus; }

int set_error(int code, const char *fmt, ...)
{
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
    const char *abort_env = getenv("COMET_HIP_ABORT_ON_ERROR");
    if (abort_env && abort_env[0] == '1') {
        fprintf(stderr, "comet_hip error %d: %s\n", code, buf);
        exit(1);
    }
    return code;
}

static int do_init(int device)
{
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
        return set_error(COMET_HIP_ERR_NOGPU, "no HIP device available (%s)",
                         e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    if (device < 0 || device >= count)
        return set_error(COMET_HIP_ERR_ARG, "device %d out of range [0,%d)", device, count);
    COMET_HIPCHK(hipSetDevice(device));
    hipDeviceProp_t prop;
    COMET_HIPCHK(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return set_error(COMET_HIP_ERR_NOGPU, "device %d is %s; this library holds gfx950 code only",
                         device, prop.gcnArchName);
    g_num_cus = prop.multiProcessorCount;
    COMET_HIPCHK(hipStreamCreate(&g_stream));
    COMET_HIPCHK(hipStreamCreate(&g_aux));
    COMET_HIPCHK(hipEventCreateWithFlags(&g_fork, hipEventDisableTiming));
    COMET_HIPCHK(hipEventCreateWithFlags(&g_join, hipEventDisableTiming));
    COMET_CHK(spmm_static_setup(device));
    g_device = device;
    g_inited = true;
    return COMET_HIP_OK;
}

bool is_initialised() { return g_inited; }

int ensure_init()
{
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_inited)
        return COMET_HIP_OK;
    return do_init(0);
}

// every workspace that ever held memory, so that comet_hip_finalize can give all of it back
static std::vector<Workspace *> g_workspaces;

int Workspace::ensure(size_t need, bool zeroed)
{
    if (need <= bytes)
        return COMET_HIP_OK;
    if (!listed) {
        g_workspaces.push_back(this);
        listed = true;
    }
    if (ptr) {
        COMET_HIPCHK(hipStreamSynchronize(stream()));
        COMET_HIPCHK(hipFree(ptr));
        ptr = nullptr;
        bytes = 0;
    }
    COMET_HIPCHK(hipMalloc(&ptr, need));
    bytes = need;
    if (zeroed)
        COMET_HIPCHK(hipMemsetAsync(ptr, 0, need, stream()));
    return COMET_HIP_OK;
}

void Workspace::release()
{
    if (ptr)
        (void)hipFree(ptr);
    ptr = nullptr;
    bytes = 0;
}

Csr *csr_from_handle(int64_t h, bool allow_poisoned)
{
    Csr *c = reinterpret_cast<Csr *>(h);
    std::lock_guard<std::mutex> lk(g_mu);
    if (!c || !g_live.count(c)) {
        set_error(COMET_HIP_ERR_HANDLE, "unknown CSR handle %lld", (long long)h);
        return nullptr;
    }
    if (c->poisoned && !allow_poisoned) {
        set_error(COMET_HIP_ERR_HANDLE,
                  "CSR handle %lld: its arrays failed the check of comet_hip_csr_invalidate; rewrite them and "
                  "invalidate again, or destroy the handle", (long long)h);
        return nullptr;
    }
    return c;
}

int64_t csr_register(Csr *c)
{
    std::lock_guard<std::mutex> lk(g_mu);
    g_live.insert(c);
    return reinterpret_cast<int64_t>(c);
}

int csr_alloc(Csr *c, int64_t nrows, int64_t ncols, int64_t nnz)
{
    c->nrows = nrows;
    c->ncols = ncols;
    c->nnz = nnz;
    c->owns = true;
    COMET_HIPCHK(hipMalloc((void **)&c->pos, sizeof(int64_t) * (size_t)(nrows + 1)));
    COMET_HIPCHK(hipMalloc((void **)&c->crd, sizeof(int32_t) * (size_t)(nnz > 0 ? nnz : 1)));
    COMET_HIPCHK(hipMalloc((void **)&c->val, sizeof(double) * (size_t)(nnz > 0 ? nnz : 1)));
    return COMET_HIP_OK;
}

// Everything the kernels derived from the matrix and keep in its handle.
bool plan_at_once()
{
    return getenv("COMET_HIP_PLAN_AT_ONCE") != nullptr;
}

uint64_t next_csr_uid()
{
    static std::atomic<uint64_t> next{1};
    return next.fetch_add(1);
}

static void csr_drop_plans(Csr *c)
{
    c->uid = next_csr_uid();
    for (auto &e : c->row_lists) {
        (void)hipFree(e.rows);
        (void)hipFree(e.bounds);
    }
    c->row_lists.clear();
    if (c->light)
        csr_release(c->light);
    if (c->transposed)
        csr_release(c->transposed);
    if (c->transposed_index)
        csr_release(c->transposed_index);
    c->light = c->transposed = c->transposed_index = nullptr;
    c->dup_state = 0;
    c->iso_state = 0;
    (void)hipFree(c->entry_row);
    c->entry_row = nullptr;
    (void)hipFree(c->rowmap);
    (void)hipFree(c->empty_rows);
    c->rowmap = c->empty_rows = nullptr;
    c->nempty = 0;
    (void)hipFree(c->heavy_seg);
    (void)hipFree(c->heavy_ent);
    (void)hipFree(c->heavy_row);
    (void)hipFree(c->heavy_code);
    (void)hipFree(c->medium_row);
    c->medium_row = nullptr;
    c->medium_rows = 0;
    c->heavy_seg = nullptr;
    c->heavy_ent = nullptr;
    c->heavy_row = c->heavy_code = nullptr;
    c->heavy_state = 0;
    c->spmm_uses = c->spmv_uses = 0;
    c->heavy_nnz = c->heavy_rows = 0;
    (void)hipFree(c->spmm_chunk_row);
    c->spmm_chunk_row = nullptr;
    c->spmm_nchunks = 0;
    (void)hipFree(c->sg_blkptr);
    (void)hipFree(c->sg_crd16);
    c->sg_blkptr = nullptr;
    c->sg_crd16 = nullptr;
    c->sg_nblk = 0;
    (void)hipFree(c->spmv_bpos);
    (void)hipFree(c->spmv_bpos32);
    c->spmv_bpos32 = nullptr;
    (void)hipFree(c->spmv_bcrd);
    (void)hipFree(c->spmv_bval);
    c->spmv_bpos = nullptr;
    c->spmv_bcrd = nullptr;
    c->spmv_bval = nullptr;
    c->spmv_nb = 0;
    c->spmv_base.clear();
}

void csr_release(Csr *c)
{
    csr_drop_plans(c);
    if (c->owns) {
        (void)hipFree(c->pos);
        (void)hipFree(c->crd);
        (void)hipFree(c->val);
    }
    delete c;
}

// ------------------------------------------------------------------ profiling
struct ProfEntry { int64_t launches = 0; double ms = 0.0; };
struct Pending { std::string name; hipEvent_t a, b; };
static bool g_prof_on = false;
static std::map<std::string, ProfEntry> g_prof;
static std::vector<Pending> g_pending;
static std::vector<hipEvent_t> g_event_pool;
static hipEvent_t g_t0 = nullptr, g_t1 = nullptr;

static hipEvent_t take_event()
{
    if (!g_event_pool.empty()) {
        hipEvent_t e = g_event_pool.back();
        g_event_pool.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    (void)hipEventCreate(&e);
    return e;
}

static void drain_pending()
{
    if (g_pending.empty())
        return;
    (void)hipStreamSynchronize(g_stream);
    (void)hipStreamSynchronize(g_aux);
    for (auto &p : g_pending) {
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, p.a, p.b) == hipSuccess) {
            auto &e = g_prof[p.name];
            e.launches += 1;
            e.ms += ms;
        }
        g_event_pool.push_back(p.a);
        g_event_pool.push_back(p.b);
    }
    g_pending.clear();
}

KernelTimer::KernelTimer(const char *name) : KernelTimer(name, g_stream) {}

KernelTimer::KernelTimer(const char *name, hipStream_t s) : slot(-1), on(s)
{
    if (!g_prof_on)
        return;
    if (g_pending.size() >= 4096)
        drain_pending();
    Pending p;
    p.name = name;
    p.a = take_event();
    p.b = take_event();
    (void)hipEventRecord(p.a, on);
    g_pending.push_back(p);
    slot = (int)g_pending.size() - 1;
}

KernelTimer::~KernelTimer()
{
    if (slot >= 0)
        (void)hipEventRecord(g_pending[slot].b, on);
}

// ------------------------------------------------------------------ kernels
__global__ void narrow_i64_to_i32(const int64_t *__restrict__ in, int32_t *__restrict__ out, int64_t n)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += step)
        out[i] = (int32_t)in[i];
}

__global__ void widen_i32_to_i64(const int32_t *__restrict__ in, int64_t *__restrict__ out, int64_t n)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += step)
        out[i] = (int64_t)in[i];
}

__global__ void copy_f64_kernel(double *__restrict__ dst, const double *__restrict__ src, int64_t n)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += step)
        dst[i] = src[i];
}

// Streaming yardsticks, 16 bytes per lane: what the memory system gives a kernel that does nothing but move bytes.
// Every workgroup walks a contiguous slice so that a DRAM page is opened by one workgroup, not by all of them.
typedef double stream_v2d __attribute__((ext_vector_type(2)));

template <bool NT>
__global__ __launch_bounds__(256) void stream_copy16_kernel(stream_v2d *__restrict__ dst, const stream_v2d *__restrict__ src,
                                                            int64_t n2)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    const auto ld = [](const stream_v2d *p) { return NT ? __builtin_nontemporal_load(p) : *p; };
    const auto st = [](stream_v2d v, stream_v2d *p) {
        if (NT)
            __builtin_nontemporal_store(v, p);
        else
            *p = v;
    };
    for (; i + 3 * step < n2; i += 4 * step) {      // four loads in flight per lane, then four stores
        const stream_v2d a = ld(src + i), b = ld(src + i + step), c = ld(src + i + 2 * step), d = ld(src + i + 3 * step);
        st(a, dst + i);
        st(b, dst + i + step);
        st(c, dst + i + 2 * step);
        st(d, dst + i + 3 * step);
    }
    for (; i < n2; i += step)
        st(ld(src + i), dst + i);
}

// read-only: every lane sums what it reads, one store per lane at the end
__global__ __launch_bounds__(256) void stream_read16_kernel(const stream_v2d *__restrict__ src, int64_t n2,
                                                            double *__restrict__ out)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    stream_v2d s0 = {0.0, 0.0}, s1 = s0, s2 = s0, s3 = s0;
    for (; i + 3 * step < n2; i += 4 * step) {
        const stream_v2d a = __builtin_nontemporal_load(src + i), b = __builtin_nontemporal_load(src + i + step),
                         c = __builtin_nontemporal_load(src + i + 2 * step),
                         d = __builtin_nontemporal_load(src + i + 3 * step);
        s0 += a;
        s1 += b;
        s2 += c;
        s3 += d;
    }
    for (; i < n2; i += step)
        s0 += __builtin_nontemporal_load(src + i);
    s0 += s1 + s2 + s3;
    out[(int64_t)blockIdx.x * blockDim.x + threadIdx.x] = s0.x + s0.y;
}

// write-only
__global__ __launch_bounds__(256) void stream_write16_kernel(stream_v2d *__restrict__ dst, int64_t n2, double v)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    const stream_v2d w = {v, v};
    for (; i < n2; i += step)
        __builtin_nontemporal_store(w, dst + i);
}

// Exclusive scan, three launches: per-block totals, scan of the totals by one
// block, then a per-block rescan with the block offset added.
constexpr int SCAN_T = 256;          // threads per block
constexpr int SCAN_E = 8;            // elements per thread
constexpr int SCAN_B = SCAN_T * SCAN_E;

__device__ inline int64_t block_exclusive_scan(int64_t v, int64_t *total, int64_t *lds /* SCAN_T/64+1 */)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int64_t inc = v;
    for (int d = 1; d < 64; d <<= 1) {
        int64_t o = __shfl_up(inc, d, 64);
        if (lane >= d)
            inc += o;
    }
    if (lane == 63)
        lds[wave] = inc;
    __syncthreads();
    int64_t wave_off = 0, tot = 0;
    const int nw = blockDim.x >> 6;
    for (int w = 0; w < nw; ++w) {
        int64_t s = lds[w];
        if (w < wave)
            wave_off += s;
        tot += s;
    }
    __syncthreads();
    *total = tot;
    return wave_off + inc - v;
}

__global__ __launch_bounds__(SCAN_T) void scan_block_totals(const int64_t *__restrict__ in, int64_t n,
                                                            int64_t *__restrict__ block_tot)
{
    __shared__ int64_t lds[SCAN_T / 64 + 1];
    int64_t base = (int64_t)blockIdx.x * SCAN_B + (int64_t)threadIdx.x * SCAN_E;
    int64_t s = 0;
    for (int e = 0; e < SCAN_E; ++e)
        if (base + e < n)
            s += in[base + e];
    int64_t tot;
    block_exclusive_scan(s, &tot, lds);
    if (threadIdx.x == 0)
        block_tot[blockIdx.x] = tot;
}

__global__ __launch_bounds__(SCAN_T) void scan_totals_inplace(int64_t *__restrict__ block_tot, int64_t nblocks)
{
    __shared__ int64_t lds[SCAN_T / 64 + 1];
    int64_t carry = 0;
    for (int64_t base = 0; base < nblocks; base += SCAN_T) {
        int64_t i = base + threadIdx.x;
        int64_t v = i < nblocks ? block_tot[i] : 0;
        int64_t tot;
        int64_t ex = block_exclusive_scan(v, &tot, lds);
        if (i < nblocks)
            block_tot[i] = carry + ex;
        carry += tot;
    }
    if (threadIdx.x == 0)
        block_tot[nblocks] = carry;
}

__global__ __launch_bounds__(SCAN_T) void scan_apply(const int64_t *__restrict__ in, int64_t n,
                                                     const int64_t *__restrict__ block_off,
                                                     int64_t nblocks, int64_t *__restrict__ pos)
{
    __shared__ int64_t lds[SCAN_T / 64 + 1];
    int64_t base = (int64_t)blockIdx.x * SCAN_B + (int64_t)threadIdx.x * SCAN_E;
    int64_t v[SCAN_E];
    int64_t s = 0;
    for (int e = 0; e < SCAN_E; ++e) {
        v[e] = base + e < n ? in[base + e] : 0;
        s += v[e];
    }
    int64_t tot;
    int64_t run = block_off[blockIdx.x] + block_exclusive_scan(s, &tot, lds);
    for (int e = 0; e < SCAN_E; ++e) {
        if (base + e < n)
            pos[base + e] = run;
        run += v[e];
    }
    if (blockIdx.x == 0 && threadIdx.x == 0)
        pos[n] = block_off[nblocks];
}

static Workspace g_scan_ws;

int exclusive_scan_i64(const int64_t *counts, int64_t n, int64_t *pos)
{
    if (n <= 0) {
        COMET_HIPCHK(hipMemsetAsync(pos, 0, sizeof(int64_t), stream()));
        return COMET_HIP_OK;
    }
    int64_t nblocks = ceil_div(n, SCAN_B);
    COMET_CHK(g_scan_ws.ensure(sizeof(int64_t) * (size_t)(nblocks + 1), false));
    int64_t *tot = (int64_t *)g_scan_ws.ptr;
    {
        KernelTimer t("scan_block_totals");
        scan_block_totals<<<dim3((unsigned)nblocks), dim3(SCAN_T), 0, stream()>>>(counts, n, tot);
    }
    {
        KernelTimer t("scan_totals_inplace");
        scan_totals_inplace<<<dim3(1), dim3(SCAN_T), 0, stream()>>>(tot, nblocks);
    }
    {
        KernelTimer t("scan_apply");
        scan_apply<<<dim3((unsigned)nblocks), dim3(SCAN_T), 0, stream()>>>(counts, n, tot, nblocks, pos);
    }
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}

// Deterministic two-level tree sum.
constexpr int RED_T = 256;
__global__ __launch_bounds__(RED_T) void reduce_partial(const double *__restrict__ v, int64_t n,
                                                        double *__restrict__ partial)
{
    __shared__ double lds[RED_T];
    double s = 0.0;
    // fixed assignment of elements to threads: independent of the grid only through gridDim, which the host fixes per n
    for (int64_t i = (int64_t)blockIdx.x * RED_T + threadIdx.x; i < n; i += (int64_t)gridDim.x * RED_T)
        s += v[i];
    lds[threadIdx.x] = s;
    __syncthreads();
    for (int d = RED_T / 2; d > 0; d >>= 1) {
        if ((int)threadIdx.x < d)
            lds[threadIdx.x] += lds[threadIdx.x + d];
        __syncthreads();
    }
    if (threadIdx.x == 0)
        partial[blockIdx.x] = lds[0];
}

static Workspace g_red_ws;

int reduce_sum_device(const double *v, int64_t n, double *out_host)
{
    if (n <= 0) {
        *out_host = 0.0;
        return COMET_HIP_OK;
    }
    int64_t nb = ceil_div(n, (int64_t)RED_T * 16);
    if (nb > 1024)
        nb = 1024;
    COMET_CHK(g_red_ws.ensure(sizeof(double) * (size_t)(nb + 1), false));
    double *partial = (double *)g_red_ws.ptr;
    {
        KernelTimer t("reduce_partial");
        reduce_partial<<<dim3((unsigned)nb), dim3(RED_T), 0, stream()>>>(v, n, partial);
    }
    {
        KernelTimer t("reduce_final");
        reduce_partial<<<dim3(1), dim3(RED_T), 0, stream()>>>(partial, nb, partial + nb);
    }
    COMET_HIPCHK(hipGetLastError());
    COMET_HIPCHK(hipMemcpyAsync(out_host, partial + nb, sizeof(double), hipMemcpyDeviceToHost, stream()));
    COMET_HIPCHK(hipStreamSynchronize(stream()));
    return COMET_HIP_OK;
}

}  // namespace comet

using namespace comet;

template <typename I>
static int validate_host_csr(int64_t nrows, int64_t ncols, const I *pos, const I *crd, const double *val)
{
    if (nrows < 0 || ncols < 0 || !pos)
        return set_error(COMET_HIP_ERR_ARG, "bad CSR dimensions or null pos");
    if (nrows >= INT32_MAX || ncols >= INT32_MAX)
        return set_error(COMET_HIP_ERR_SIZE, "CSR dimensions %lld x %lld exceed the int32 column index",
                         (long long)nrows, (long long)ncols);
    if (pos[0] != 0)
        return set_error(COMET_HIP_ERR_ARG, "pos[0] = %lld, expected 0", (long long)pos[0]);
    for (int64_t i = 0; i < nrows; ++i)
        if (pos[i + 1] < pos[i])
            return set_error(COMET_HIP_ERR_ARG, "pos not monotone at row %lld", (long long)i);
    int64_t nnz = (int64_t)pos[nrows];
    if (nnz > 0 && (!crd || !val))
        return set_error(COMET_HIP_ERR_ARG, "null crd/val with nnz = %lld", (long long)nnz);
    for (int64_t p = 0; p < nnz; ++p)
        if (crd[p] < 0 || (int64_t)crd[p] >= ncols)
            return set_error(COMET_HIP_ERR_ARG, "crd[%lld] = %lld outside [0,%lld)", (long long)p,
                             (long long)crd[p], (long long)ncols);
    // The kernels bisect rows and index on-chip windows with (column - window start): a row whose columns
    // go down would put entries outside those windows.  Equal neighbours (duplicates) are fine.
    for (int64_t i = 0; i < nrows; ++i)
        for (int64_t p = (int64_t)pos[i] + 1; p < (int64_t)pos[i + 1]; ++p)
            if (crd[p] < crd[p - 1])
                return set_error(COMET_HIP_ERR_ARG,
                                 "row %lld: column %lld follows column %lld; the columns of a row must not decrease "
                                 "(comet_hip_csr_from_coo_i64 orders tuples)",
                                 (long long)i, (long long)crd[p], (long long)crd[p - 1]);
    return COMET_HIP_OK;
}

// The same checks for arrays that already sit in HBM: one wavefront per row.  *bad becomes non-zero if pos does
// not start at 0, decreases, does not end at nnz, or a column is out of range or smaller than its left neighbour.
__global__ __launch_bounds__(256) void csr_check_device(int64_t nrows, int64_t ncols, int64_t nnz,
                                                        const int64_t *__restrict__ pos,
                                                        const int32_t *__restrict__ crd, int32_t *__restrict__ bad)
{
    const int lane = threadIdx.x & 63;
    const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
    if (wave == 0 && lane == 0 && (pos[0] != 0 || pos[nrows] != nnz))
        *bad = 1;
    for (int64_t r = wave; r < nrows; r += nwaves) {
        const int64_t s = pos[r], e = pos[r + 1];
        if (s < 0 || e < s || e > nnz) {        // entries of such a row are not touched
            if (lane == 0)
                *bad = 1;
            continue;
        }
        for (int64_t p = s + lane; p < e; p += 64) {
            const int32_t c = crd[p];
            if (c < 0 || c >= ncols || (p > s && c < crd[p - 1]))
                *bad = 1;
        }
    }
}

static Workspace g_check_flag;

static int validate_device_csr(const Csr *c)
{
    COMET_CHK(g_check_flag.ensure(sizeof(int32_t), false));
    int32_t *flag = (int32_t *)g_check_flag.ptr;
    COMET_HIPCHK(hipMemsetAsync(flag, 0, sizeof(int32_t), stream()));
    const unsigned blocks = (unsigned)std::min<int64_t>(std::max<int64_t>(ceil_div(c->nrows, 4), 1), 16384);
    csr_check_device<<<dim3(blocks), dim3(256), 0, stream()>>>(c->nrows, c->ncols, c->nnz, c->pos, c->crd, flag);
    COMET_HIPCHK(hipGetLastError());
    int32_t bad = 0;
    COMET_HIPCHK(hipMemcpyAsync(&bad, flag, sizeof(int32_t), hipMemcpyDeviceToHost, stream()));
    COMET_HIPCHK(hipStreamSynchronize(stream()));
    if (bad)
        return set_error(COMET_HIP_ERR_ARG,
                         "device CSR arrays are not a valid matrix: pos must start at 0, never decrease and end at nnz; "
                         "columns must lie in [0, ncols) and must not decrease inside a row");
    return COMET_HIP_OK;
}


// ====================================================================== C ABI
extern "C" {

int comet_hip_init(int device)
{
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_inited) {
        if (device != g_device)
            return set_error(COMET_HIP_ERR_ARG, "already initialised on device %d", g_device);
        return COMET_HIP_OK;
    }
    return do_init(device);
}

int comet_hip_finalize(void)
{
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_inited)
        return COMET_HIP_OK;
    (void)hipStreamSynchronize(g_stream);
    forget_pending_reads();       // handles kept between a "sizes" call and its "fill" call die with the rest
    forget_pending_product();
    for (Csr *c : g_live)
        csr_release(c);
    g_live.clear();
    for (Workspace *w : g_workspaces)
        w->release();
    (void)hipStreamSynchronize(g_aux);
    (void)hipEventDestroy(g_fork);
    (void)hipEventDestroy(g_join);
    (void)hipStreamDestroy(g_aux);
    (void)hipStreamDestroy(g_stream);
    g_stream = g_aux = nullptr;
    g_fork = g_join = nullptr;
    g_inited = false;
    return COMET_HIP_OK;
}

const char *comet_hip_last_error(void) { return g_last_error.c_str(); }

int comet_hip_device_name(char *buf, int64_t cap)
{
    COMET_CHK(ensure_init());
    if (!buf || cap <= 0)
        return set_error(COMET_HIP_ERR_ARG, "null buffer");
    hipDeviceProp_t prop;
    COMET_HIPCHK(hipGetDeviceProperties(&prop, g_device));
    snprintf(buf, (size_t)cap, "%s (%s, %d CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
    return COMET_HIP_OK;
}

int64_t comet_hip_malloc(int64_t bytes)
{
    if (ensure_init() != COMET_HIP_OK)
        return 0;
    if (bytes < 0) {
        set_error(COMET_HIP_ERR_ARG, "negative allocation size %lld", (long long)bytes);
        return 0;
    }
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, (size_t)(bytes > 0 ? bytes : 1));
    if (e != hipSuccess) {
        set_error(COMET_HIP_ERR_HIP, "hipMalloc(%lld) failed: %s", (long long)bytes, hipGetErrorString(e));
        return 0;
    }
    return (int64_t)p;
}

int comet_hip_free(int64_t dptr)
{
    COMET_CHK(ensure_init());
    if (!dptr)
        return COMET_HIP_OK;
    COMET_HIPCHK(hipStreamSynchronize(stream()));
    COMET_HIPCHK(hipFree((void *)dptr));
    return COMET_HIP_OK;
}

int comet_hip_memcpy(int64_t dptr, void *host, int64_t bytes, int64_t direction)
{
    COMET_CHK(ensure_init());
    if (bytes < 0 || (bytes > 0 && (!dptr || !host)))
        return set_error(COMET_HIP_ERR_ARG, "bad memcpy arguments");
    if (bytes == 0)
        return COMET_HIP_OK;
    if (direction == 0)
        COMET_HIPCHK(hipMemcpyAsync((void *)dptr, host, (size_t)bytes, hipMemcpyHostToDevice, stream()));
    else
        COMET_HIPCHK(hipMemcpyAsync(host, (void *)dptr, (size_t)bytes, hipMemcpyDeviceToHost, stream()));
    COMET_HIPCHK(hipStreamSynchronize(stream()));
    return COMET_HIP_OK;
}

int comet_hip_memset(int64_t dptr, int byte_value, int64_t bytes)
{
    COMET_CHK(ensure_init());
    if (bytes < 0 || (bytes > 0 && !dptr))
        return set_error(COMET_HIP_ERR_ARG, "bad memset arguments");
    if (bytes)
        COMET_HIPCHK(hipMemsetAsync((void *)dptr, byte_value, (size_t)bytes, stream()));
    return COMET_HIP_OK;
}

int comet_hip_sync(void)
{
    COMET_CHK(ensure_init());
    COMET_HIPCHK(hipStreamSynchronize(stream()));
    return COMET_HIP_OK;
}

// Names and argument lists of the reference glue, kept so lowered code that
// still allocates and copies through them links unchanged.
int64_t HipMallocF64(int64_t n) { return comet_hip_malloc(n * 8); }
int64_t HipMallocI64(int64_t n) { return comet_hip_malloc(n * 8); }
int64_t HipMallocI32(int64_t n) { return comet_hip_malloc(n * 4); }
void HipFree(int64_t dptr) { (void)comet_hip_free(dptr); }
void HipMemcpyF64(int64_t dptr, void *, void *aligned, int64_t offset, int64_t size, int64_t, int64_t dir)
{
    (void)comet_hip_memcpy(dptr, (double *)aligned + offset, size * 8, dir);
}
void HipMemcpyI64(int64_t dptr, void *, void *aligned, int64_t offset, int64_t size, int64_t, int64_t dir)
{
    (void)comet_hip_memcpy(dptr, (int64_t *)aligned + offset, size * 8, dir);
}
void HipMemcpyI32(int64_t dptr, void *, void *aligned, int64_t offset, int64_t size, int64_t, int64_t dir)
{
    (void)comet_hip_memcpy(dptr, (int32_t *)aligned + offset, size * 4, dir);
}
void HipMemcpyIndex(int64_t dptr, void *p, void *aligned, int64_t offset, int64_t size, int64_t stride, int64_t dir)
{
    HipMemcpyI64(dptr, p, aligned, offset, size, stride, dir);
}

// ------------------------------------------------------------------ CSR
int64_t comet_hip_csr_upload_i64(int64_t nrows, int64_t ncols, const int64_t *pos, const int64_t *crd,
                                 const double *val)
{
    if (ensure_init() != COMET_HIP_OK)
        return 0;
    if (validate_host_csr(nrows, ncols, pos, crd, val) != COMET_HIP_OK)
        return 0;
    int64_t nnz = pos[nrows];
    Csr *c = new Csr();
    int64_t *tmp = nullptr;
    auto fail = [&]() -> int64_t {
        if (tmp)
            (void)hipFree(tmp);
        csr_release(c);
        return 0;
    };
    if (csr_alloc(c, nrows, ncols, nnz) != COMET_HIP_OK)
        return fail();
    hipStream_t s = stream();
    if (hipMemcpyAsync(c->pos, pos, sizeof(int64_t) * (size_t)(nrows + 1), hipMemcpyHostToDevice, s) != hipSuccess)
        return set_error(COMET_HIP_ERR_HIP, "pos upload failed"), fail();
    if (nnz > 0) {
        if (hipMalloc((void **)&tmp, sizeof(int64_t) * (size_t)nnz) != hipSuccess)
            return set_error(COMET_HIP_ERR_HIP, "staging allocation failed"), fail();
        if (hipMemcpyAsync(tmp, crd, sizeof(int64_t) * (size_t)nnz, hipMemcpyHostToDevice, s) != hipSuccess ||
            hipMemcpyAsync(c->val, val, sizeof(double) * (size_t)nnz, hipMemcpyHostToDevice, s) != hipSuccess)
            return set_error(COMET_HIP_ERR_HIP, "crd/val upload failed"), fail();
        unsigned blocks = (unsigned)std::min<int64_t>(ceil_div(nnz, 256), 65536);
        narrow_i64_to_i32<<<dim3(blocks), dim3(256), 0, s>>>(tmp, c->crd, nnz);
    }
    if (hipStreamSynchronize(s) != hipSuccess)
        return set_error(COMET_HIP_ERR_HIP, "upload synchronisation failed"), fail();
    if (tmp)
        (void)hipFree(tmp);
    return csr_register(c);
}

int64_t comet_hip_csr_upload_i32(int64_t nrows, int64_t ncols, const int32_t *pos, const int32_t *crd,
                                 const double *val)
{
    if (ensure_init() != COMET_HIP_OK)
        return 0;
    if (validate_host_csr(nrows, ncols, pos, crd, val) != COMET_HIP_OK)
        return 0;
    int64_t nnz = pos[nrows];
    Csr *c = new Csr();
    int32_t *tmp = nullptr;
    auto fail = [&]() -> int64_t {
        if (tmp)
            (void)hipFree(tmp);
        csr_release(c);
        return 0;
    };
    if (csr_alloc(c, nrows, ncols, nnz) != COMET_HIP_OK)
        return fail();
    hipStream_t s = stream();
    if (hipMalloc((void **)&tmp, sizeof(int32_t) * (size_t)(nrows + 1)) != hipSuccess)
        return set_error(COMET_HIP_ERR_HIP, "staging allocation failed"), fail();
    if (hipMemcpyAsync(tmp, pos, sizeof(int32_t) * (size_t)(nrows + 1), hipMemcpyHostToDevice, s) != hipSuccess)
        return set_error(COMET_HIP_ERR_HIP, "pos upload failed"), fail();
    unsigned blocks = (unsigned)std::min<int64_t>(ceil_div(nrows + 1, 256), 65536);
    widen_i32_to_i64<<<dim3(blocks), dim3(256), 0, s>>>(tmp, c->pos, nrows + 1);
    if (nnz > 0) {
        if (hipMemcpyAsync(c->crd, crd, sizeof(int32_t) * (size_t)nnz, hipMemcpyHostToDevice, s) != hipSuccess ||
            hipMemcpyAsync(c->val, val, sizeof(double) * (size_t)nnz, hipMemcpyHostToDevice, s) != hipSuccess)
            return set_error(COMET_HIP_ERR_HIP, "crd/val upload failed"), fail();
    }
    if (hipStreamSynchronize(s) != hipSuccess)
        return set_error(COMET_HIP_ERR_HIP, "upload synchronisation failed"), fail();
    (void)hipFree(tmp);
    return csr_register(c);
}

int64_t comet_hip_csr_wrap(int64_t nrows, int64_t ncols, int64_t nnz, int64_t pos_dptr, int64_t crd_dptr,
                           int64_t val_dptr)
{
    if (ensure_init() != COMET_HIP_OK)
        return 0;
    if (nrows < 0 || ncols < 0 || nnz < 0 || !pos_dptr || (nnz > 0 && (!crd_dptr || !val_dptr)) ||
        nrows >= INT32_MAX || ncols >= INT32_MAX) {
        set_error(COMET_HIP_ERR_ARG, "bad arguments to comet_hip_csr_wrap");
        return 0;
    }
    Csr *c = new Csr();
    c->nrows = nrows;
    c->ncols = ncols;
    c->nnz = nnz;
    c->pos = (int64_t *)pos_dptr;
    c->crd = (int32_t *)crd_dptr;
    c->val = (double *)val_dptr;
    c->owns = false;
    // an out-of-range column or row pointer would send the kernels outside their buffers: look once, now
    if (validate_device_csr(c) != COMET_HIP_OK) {
        csr_release(c);
        return 0;
    }
    return csr_register(c);
}

int comet_hip_csr_dims(int64_t csr, int64_t *nrows, int64_t *ncols, int64_t *nnz)
{
    Csr *c = csr_from_handle(csr);
    if (!c)
        return COMET_HIP_ERR_HANDLE;
    if (nrows) *nrows = c->nrows;
    if (ncols) *ncols = c->ncols;
    if (nnz) *nnz = c->nnz;
    return COMET_HIP_OK;
}

int comet_hip_csr_arrays(int64_t csr, int64_t *pos_dptr, int64_t *crd_dptr, int64_t *val_dptr)
{
    Csr *c = csr_from_handle(csr);
    if (!c)
        return COMET_HIP_ERR_HANDLE;
    if (pos_dptr) *pos_dptr = (int64_t)c->pos;
    if (crd_dptr) *crd_dptr = (int64_t)c->crd;
    if (val_dptr) *val_dptr = (int64_t)c->val;
    return COMET_HIP_OK;
}

int comet_hip_csr_download_i64(int64_t csr, int64_t *pos, int64_t *crd, double *val)
{
    Csr *c = csr_from_handle(csr);
    if (!c)
        return COMET_HIP_ERR_HANDLE;
    hipStream_t s = stream();
    if (pos)
        COMET_HIPCHK(hipMemcpyAsync(pos, c->pos, sizeof(int64_t) * (size_t)(c->nrows + 1), hipMemcpyDeviceToHost, s));
    if (val && c->nnz)
        COMET_HIPCHK(hipMemcpyAsync(val, c->val, sizeof(double) * (size_t)c->nnz, hipMemcpyDeviceToHost, s));
    if (crd && c->nnz) {
        int64_t *tmp = nullptr;
        COMET_HIPCHK(hipMalloc((void **)&tmp, sizeof(int64_t) * (size_t)c->nnz));
        unsigned blocks = (unsigned)std::min<int64_t>(ceil_div(c->nnz, 256), 65536);
        widen_i32_to_i64<<<dim3(blocks), dim3(256), 0, s>>>(c->crd, tmp, c->nnz);
        hipError_t e = hipMemcpyAsync(crd, tmp, sizeof(int64_t) * (size_t)c->nnz, hipMemcpyDeviceToHost, s);
        hipError_t e2 = hipStreamSynchronize(s);
        (void)hipFree(tmp);
        COMET_HIPCHK(e);
        COMET_HIPCHK(e2);
    }
    COMET_HIPCHK(hipStreamSynchronize(s));
    return COMET_HIP_OK;
}

int comet_hip_csr_download_i32(int64_t csr, int32_t *pos, int32_t *crd, double *val)
{
    Csr *c = csr_from_handle(csr);
    if (!c)
        return COMET_HIP_ERR_HANDLE;
    if (pos && c->nnz > INT32_MAX)
        return set_error(COMET_HIP_ERR_SIZE, "nnz %lld does not fit an int32 row pointer", (long long)c->nnz);
    hipStream_t s = stream();
    if (pos) {
        int32_t *tmp = nullptr;
        COMET_HIPCHK(hipMalloc((void **)&tmp, sizeof(int32_t) * (size_t)(c->nrows + 1)));
        unsigned blocks = (unsigned)std::min<int64_t>(ceil_div(c->nrows + 1, 256), 65536);
        narrow_i64_to_i32<<<dim3(blocks), dim3(256), 0, s>>>(c->pos, tmp, c->nrows + 1);
        hipError_t e = hipMemcpyAsync(pos, tmp, sizeof(int32_t) * (size_t)(c->nrows + 1), hipMemcpyDeviceToHost, s);
        hipError_t e2 = hipStreamSynchronize(s);
        (void)hipFree(tmp);
        COMET_HIPCHK(e);
        COMET_HIPCHK(e2);
    }
    if (crd && c->nnz)
        COMET_HIPCHK(hipMemcpyAsync(crd, c->crd, sizeof(int32_t) * (size_t)c->nnz, hipMemcpyDeviceToHost, s));
    if (val && c->nnz)
        COMET_HIPCHK(hipMemcpyAsync(val, c->val, sizeof(double) * (size_t)c->nnz, hipMemcpyDeviceToHost, s));
    COMET_HIPCHK(hipStreamSynchronize(s));
    return COMET_HIP_OK;
}

int comet_hip_csr_invalidate(int64_t csr)
{
    Csr *c = csr_from_handle(csr, true);
    if (!c)
        return COMET_HIP_ERR_HANDLE;
    COMET_HIPCHK(hipStreamSynchronize(stream()));
    csr_drop_plans(c);
    // the arrays were rewritten: they are looked at again, and a handle that fails is refused by every entry
    // point that would read them (out-of-range columns fault the GPU) until a later call here passes
    const int rc = validate_device_csr(c);
    c->poisoned = rc != COMET_HIP_OK;
    return rc;
}

int comet_hip_csr_destroy(int64_t csr)
{
    Csr *c = csr_from_handle(csr, true);
    if (!c)
        return COMET_HIP_ERR_HANDLE;
    COMET_HIPCHK(hipStreamSynchronize(stream()));
    {
        std::lock_guard<std::mutex> lk(g_mu);
        g_live.erase(c);
    }
    csr_release(c);
    return COMET_HIP_OK;
}

// ------------------------------------------------------------------ reduce / copy / timing
int comet_hip_reduce_sum_f64(int64_t dptr, int64_t n, double *out)
{
    COMET_CHK(ensure_init());
    if (!out || n < 0 || (n > 0 && !dptr))
        return set_error(COMET_HIP_ERR_ARG, "bad arguments to comet_hip_reduce_sum_f64");
    return comet::reduce_sum_device((const double *)dptr, n, out);
}

int comet_hip_mem_info(int64_t *free_bytes, int64_t *total_bytes)
{
    COMET_CHK(ensure_init());
    size_t f = 0, t = 0;
    COMET_HIPCHK(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = (int64_t)f;
    if (total_bytes) *total_bytes = (int64_t)t;
    return COMET_HIP_OK;
}

int comet_hip_copy_f64(int64_t dst_dptr, int64_t src_dptr, int64_t n)
{
    COMET_CHK(ensure_init());
    if (n < 0 || (n > 0 && (!dst_dptr || !src_dptr)))
        return set_error(COMET_HIP_ERR_ARG, "bad arguments to comet_hip_copy_f64");
    if (n == 0)
        return COMET_HIP_OK;
    unsigned blocks = (unsigned)std::min<int64_t>(ceil_div(n, 256), (int64_t)num_cus() * 32);
    {
        KernelTimer t("copy_f64_kernel");
        copy_f64_kernel<<<dim3(blocks), dim3(256), 0, stream()>>>((double *)dst_dptr, (const double *)src_dptr, n);
    }
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}

static Workspace g_stream_out;

// mode 0: copy, 16 bytes per lane, ordinary loads and stores; 1: the same with non-temporal loads and stores;
// 2: read only (src); 3: write only (dst).  n doubles, even; workgroups_per_cu 0 = 8.
int comet_hip_stream_bench(int mode, int64_t dst_dptr, int64_t src_dptr, int64_t n, int workgroups_per_cu)
{
    COMET_CHK(ensure_init());
    if (n <= 0 || (n & 1) || mode < 0 || mode > 3 || (mode != 2 && !dst_dptr) || (mode != 3 && !src_dptr) ||
        workgroups_per_cu < 0 || workgroups_per_cu > 64 || ((dst_dptr | src_dptr) & 15))
        return set_error(COMET_HIP_ERR_ARG, "bad arguments to comet_hip_stream_bench");
    const int64_t n2 = n / 2;
    const unsigned blocks =
        (unsigned)std::min<int64_t>(ceil_div(n2, 256), (int64_t)num_cus() * (workgroups_per_cu ? workgroups_per_cu : 8));
    if (mode == 2)
        COMET_CHK(g_stream_out.ensure(sizeof(double) * 256 * (size_t)blocks, false));
    if (mode == 0) {
        KernelTimer t("stream_copy16_kernel");
        stream_copy16_kernel<false><<<dim3(blocks), dim3(256), 0, stream()>>>((stream_v2d *)dst_dptr,
                                                                               (const stream_v2d *)src_dptr, n2);
    } else if (mode == 1) {
        KernelTimer t("stream_copy16_nt_kernel");
        stream_copy16_kernel<true><<<dim3(blocks), dim3(256), 0, stream()>>>((stream_v2d *)dst_dptr,
                                                                              (const stream_v2d *)src_dptr, n2);
    } else if (mode == 2) {
        KernelTimer t("stream_read16_kernel");
        stream_read16_kernel<<<dim3(blocks), dim3(256), 0, stream()>>>((const stream_v2d *)src_dptr, n2,
                                                                        (double *)g_stream_out.ptr);
    } else {
        KernelTimer t("stream_write16_kernel");
        stream_write16_kernel<<<dim3(blocks), dim3(256), 0, stream()>>>((stream_v2d *)dst_dptr, n2, 1.0);
    }
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}

// A stream of the caller's own (default priority), for the entry points that take one.
int64_t comet_hip_stream_create(void)
{
    if (ensure_init() != COMET_HIP_OK)
        return 0;
    hipStream_t s = nullptr;
    if (hipStreamCreateWithFlags(&s, hipStreamNonBlocking) != hipSuccess) {
        (void)hipGetLastError();
        set_error(COMET_HIP_ERR_HIP, "hipStreamCreateWithFlags failed");
        return 0;
    }
    return (int64_t)s;
}

int comet_hip_stream_sync(int64_t s)
{
    COMET_CHK(ensure_init());
    COMET_HIPCHK(hipStreamSynchronize(s ? (hipStream_t)s : stream()));
    return COMET_HIP_OK;
}

int comet_hip_stream_destroy(int64_t s)
{
    COMET_CHK(ensure_init());
    if (!s)
        return set_error(COMET_HIP_ERR_ARG, "comet_hip_stream_destroy: null stream");
    COMET_HIPCHK(hipStreamDestroy((hipStream_t)s));
    return COMET_HIP_OK;
}

int comet_hip_timer_start(void)
{
    COMET_CHK(ensure_init());
    if (!g_t0) {
        COMET_HIPCHK(hipEventCreate(&g_t0));
        COMET_HIPCHK(hipEventCreate(&g_t1));
    }
    COMET_HIPCHK(hipEventRecord(g_t0, stream()));
    return COMET_HIP_OK;
}

int comet_hip_timer_stop(double *ms)
{
    COMET_CHK(ensure_init());
    if (!g_t0 || !ms)
        return set_error(COMET_HIP_ERR_ARG, "timer_stop without timer_start");
    COMET_HIPCHK(hipEventRecord(g_t1, stream()));
    COMET_HIPCHK(hipEventSynchronize(g_t1));
    float f = 0.f;
    COMET_HIPCHK(hipEventElapsedTime(&f, g_t0, g_t1));
    *ms = f;
    return COMET_HIP_OK;
}

int comet_hip_profile_enable(int on)
{
    COMET_CHK(ensure_init());
    drain_pending();
    g_prof_on = on != 0;
    return COMET_HIP_OK;
}

int comet_hip_profile_reset(void)
{
    COMET_CHK(ensure_init());
    drain_pending();
    g_prof.clear();
    return COMET_HIP_OK;
}

int comet_hip_profile_query(const char *name, int64_t *launches, double *total_ms)
{
    COMET_CHK(ensure_init());
    drain_pending();
    if (!name) {
        if (launches) *launches = (int64_t)g_prof.size();
        if (total_ms) *total_ms = 0.0;
        return COMET_HIP_OK;
    }
    auto it = g_prof.find(name);
    if (launches) *launches = it == g_prof.end() ? 0 : it->second.launches;
    if (total_ms) *total_ms = it == g_prof.end() ? 0.0 : it->second.ms;
    return COMET_HIP_OK;
}

int comet_hip_profile_name(int32_t index, char *buf, int64_t cap)
{
    COMET_CHK(ensure_init());
    drain_pending();
    if (!buf || cap <= 0 || index < 0 || (size_t)index >= g_prof.size())
        return set_error(COMET_HIP_ERR_ARG, "bad profile index");
    auto it = g_prof.begin();
    std::advance(it, index);
    snprintf(buf, (size_t)cap, "%s", it->first.c_str());
    return COMET_HIP_OK;
}

}  // extern "C"
