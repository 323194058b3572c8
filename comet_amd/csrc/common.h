// Shared host-side plumbing of the gfx950 runtime: error reporting, the
// library stream, CSR handles, cached workspaces and per-kernel event timing.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>
#include <vector>

#include "../../include/comet_hip_rt.h"

namespace comet {

// One process-wide stream at default priority; every kernel and copy of the
// library is ordered on it.
hipStream_t stream();
// A second stream for a kernel that may run beside the one on stream(): aux_fork makes it wait for what
// stream() holds so far, aux_join makes stream() wait for it.  Both streams have the default priority.
hipStream_t aux_stream();
int aux_fork();
int aux_join();
int ensure_init();
// looks up, for `device` (current), the address of the array the allocation-free SpMM keeps its scratch in
int spmm_static_setup(int device);
bool is_initialised();     // has any call brought the device up yet
int set_error(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int num_cus();
// comet_hip_finalize destroys every handle: the two places that keep one between calls drop theirs
void forget_pending_reads();       // formats.hip: reader "sizes" call -> "read" call
void forget_pending_product();     // ciface.hip: SpGEMM "sizes" call -> "fill" call

#define COMET_HIPCHK(call)                                                                   \
    do {                                                                                     \
        hipError_t e_ = (call);                                                              \
        if (e_ != hipSuccess)                                                                \
            return comet::set_error(COMET_HIP_ERR_HIP, "%s failed: %s (%s:%d)", #call,       \
                                    hipGetErrorString(e_), __FILE__, __LINE__);              \
    } while (0)

#define COMET_CHK(expr)                \
    do {                               \
        int rc_ = (expr);              \
        if (rc_ != COMET_HIP_OK)       \
            return rc_;                \
    } while (0)

// Grow-only device scratch buffer.  `zeroed` buffers are cleared when they are
// (re)allocated and their users must leave them all-zero on return.
struct Workspace {
    void *ptr = nullptr;
    size_t bytes = 0;
    bool listed = false;
    int ensure(size_t need, bool zeroed);
    void release();
};

// One entry of the lists the SpMM sweep reads (16 bytes, one load).
struct HeavyEnt {
    int32_t ent;        // column, flags and the owned row the value adds to (see spmm_heavy_sweep)
    int32_t row;        // row of C the product is stored to, for a row with a single nonzero
    double val;
};

// A list of the rows of a product that have work, by descending number of products (what the SpGEMM kernels draw
// their tickets over), kept in the left operand's handle: it depends only on the two structures, the row range and
// the thresholds, so the seven lists a product of the benchmark takes are built once, not once per product.
struct RowListEntry {
    uint64_t b_uid = 0, mask_uid = 0, filter_uid = 0;
    int64_t rb = 0, re = 0, dense_threshold = 0, wide_threshold = 0, mask_fill = 0, xlo = 0, xhi = 0;
    int strict = 0;
    int32_t *rows = nullptr;     // device, re - rb entries
    int64_t *bounds = nullptr;   // device, 3 entries
};
uint64_t next_csr_uid();

struct Csr {
    // names this state of the matrix: new for every matrix and again whenever its arrays may have changed
    // (comet_hip_csr_invalidate), so that what other handles keep about it can tell that it is stale
    uint64_t uid = next_csr_uid();
    std::vector<RowListEntry> row_lists;
    int64_t nrows = 0, ncols = 0, nnz = 0;
    int64_t *pos = nullptr;
    int32_t *crd = nullptr;
    double *val = nullptr;
    bool owns = false;
    bool poisoned = false;      // a re-validation after comet_hip_csr_invalidate refused the arrays: no kernel may read them
    // SpMM plan: row that holds the first nonzero of every fixed-size chunk.
    int32_t *spmm_chunk_row = nullptr;
    int64_t spmm_nchunks = 0;
    // SpMV plan: the matrix re-stored as `spmv_nb` column blocks (block-major copy of crd/val, one row
    // pointer array per block) so that the slice of x a pass gathers from stays inside one L2.
    // spmv_nb == 0: not decided yet; 1: run on the original arrays.
    int spmv_nb = 0;
    int64_t *spmv_bpos = nullptr;            // [spmv_nb][nrows + 1], relative to the block's base
    int32_t *spmv_bpos32 = nullptr;          // the same in 32 bits (then spmv_bpos is null): what the passes read
    int32_t *spmv_bcrd = nullptr;
    double *spmv_bval = nullptr;
    std::vector<int64_t> spmv_base;          // first entry of each block in spmv_bcrd / spmv_bval
    // SpGEMM plan for the right-hand operand: sg_blkptr[k * (sg_nblk + 1) + cb] = position of the first entry
    // of row k whose column is >= cb * 2^14, so that the slice of a row inside one block of 16384 columns is
    // found without searching.
    int64_t *sg_blkptr = nullptr;
    int sg_nblk = 0;
    uint16_t *sg_crd16 = nullptr;            // the columns inside their block of 2^14 (null: not kept)
    // SpMM plan for long rows (heavy_state: 0 undecided, 1 not worth it, 2 in use): the long rows re-stored as
    // per-(XCD, wavefront) lists ordered by column for spmm_heavy_sweep, and the rest of the matrix as `light`.
    int heavy_state = 0;
    int64_t heavy_nnz = 0;
    int64_t *heavy_seg = nullptr;            // [8 * 512 + 1] list boundaries
    HeavyEnt *heavy_ent = nullptr;           // the lists, runs padded to even length
    int64_t heavy_rows = 0;
    int heavy_groups = 0;                    // workgroups of the sweep per XCD the lists were made for
    // rows of middling length that ride on the sweep with their sums in LDS: row m of the list is kept by workgroup
    // m % heavy_groups of every XCD in slot m / heavy_groups
    int64_t medium_rows = 0;
    int32_t *medium_row = nullptr;           // [medium_rows] row ids
    int32_t *heavy_row = nullptr;            // [heavy_rows] row ids of the long rows
    int32_t *heavy_code = nullptr;           // [8][heavy_rows] wavefront * 8 + slot that holds the row on each XCD
    Csr *light = nullptr;
    // only in a `light` matrix: it lists some rows of the product only, row r of pos being row rowmap[r] of C
    int32_t *rowmap = nullptr;
    // rows of the original that store nothing (the product clears them when it does not accumulate)
    int32_t *empty_rows = nullptr;
    int64_t nempty = 0;
    // entry_row[p] = the row that holds stored entry p (built on first use by csr_entry_rows)
    int32_t *entry_row = nullptr;
    // the transpose, built the first time a dense-times-sparse product needs it
    Csr *transposed = nullptr;
    // the transpose of the structure with, as values, the place of every entry in this matrix (a mask's, for masked
    // products taken pair by pair); dup_state: 0 not looked at, 1 no row holds a column twice, 2 some row does
    Csr *transposed_index = nullptr;
    int dup_state = 0;
    // whether all stored values are the same number (a pattern matrix, as graph kernels use them): 0 not looked
    // at, 1 they are (iso_value), 2 they are not
    int iso_state = 0;
    double iso_value = 0.0;
    // products taken with this matrix on the left so far (0, 1, more): the SpMM and SpMV plans, which cost tens of
    // products, are built when a matrix is multiplied for the second time (plan_at_once() builds them at the first)
    int spmm_uses = 0, spmv_uses = 0;
};

Csr *csr_from_handle(int64_t h, bool allow_poisoned = false);           // nullptr (and error set) if unknown
int64_t csr_register(Csr *c);              // takes ownership of the struct
int csr_alloc(Csr *c, int64_t nrows, int64_t ncols, int64_t nnz);   // allocates pos/crd/val, owns = true
void csr_release(Csr *c);                  // frees the arrays it owns, its plans and the struct
bool plan_at_once();                       // COMET_HIP_PLAN_AT_ONCE is set
int csr_entry_rows(Csr *a, const int32_t **rows);      // the row of every stored entry, kept in the handle
Csr *csr_transposed_copy(const Csr *a);    // new unregistered struct holding the transpose (nullptr on failure)

// Records an event pair around a kernel launch when profiling is on.
struct KernelTimer {
    explicit KernelTimer(const char *name);
    KernelTimer(const char *name, hipStream_t on);      // for a launch on aux_stream()
    ~KernelTimer();
    int slot;
    hipStream_t on;
};

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// exclusive scan of int64 counts into pos[0..n] (pos[n] = total), on the stream
int exclusive_scan_i64(const int64_t *counts, int64_t n, int64_t *pos);

// stable radix sort of n (key, payload) pairs on the stream, comparing key bits [0, end_bit)
int sort_pairs_u64_u32(const uint64_t *keys_in, uint64_t *keys_out, const uint32_t *vals_in, uint32_t *vals_out,
                       int64_t n, int end_bit);

// deterministic tree sum of a device array, result copied to the host
int reduce_sum_device(const double *v, int64_t n, double *out_host);

}  // namespace comet
