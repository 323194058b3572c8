/*
 * comet_hip_rt.h -- C ABI of the MI355X (gfx950) device runtime and kernel
 * library for the kernels COMET's index-tree dialect lowers to.
 *
 * Lowered COMET host code calls these entry points where it used to run the
 * generated scf loop nests (CPU) or launch Triton-generated kernels through the
 * Hip* glue (GPU).  Conventions follow that glue
 * (lib/ExecutionEngine/HipGpuUtils.cpp:31-159 in pnnl/COMET):
 *   - device buffers are opaque int64 handles that hold a device address;
 *   - host tensors arrive as memref descriptors (the `_mlir_ciface_` forms at
 *     the end of this file) or as plain pointers + sizes;
 *   - everything runs on one process-wide HIP stream owned by the library.
 * Unlike the reference glue, which prints and exit(1)s on any HIP error
 * (HipGpuUtils.cpp:10-19), every function returns a status (0 = success) and
 * keeps a message for comet_hip_last_error(); setting the environment variable
 * COMET_HIP_ABORT_ON_ERROR=1 restores print-and-exit.
 *
 * Device layout of a CSR matrix: pos int64[nrows+1], crd int32[nnz] (the index
 * width the reference selects for GPU targets, frontends/comet_dsl/comet.cpp:
 * 816-823), val float64[nnz]; columns ascending inside each row.  This is the
 * A2pos/A2crd/Aval part of the reference's sparse-tensor tuple
 * (lib/Conversion/TensorAlgebraToSCF/SparseTensorConversionPass.cpp:1281-1333).
 * Dense operands are contiguous row-major float64.
 */
#ifndef COMET_HIP_RT_H
#define COMET_HIP_RT_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define COMET_HIP_OK 0
#define COMET_HIP_ERR_ARG 1      /* null / negative / inconsistent argument      */
#define COMET_HIP_ERR_HIP 2      /* a HIP call failed                            */
#define COMET_HIP_ERR_HANDLE 3   /* unknown or already destroyed handle          */
#define COMET_HIP_ERR_SIZE 4     /* size overflows what the kernels index with   */
#define COMET_HIP_ERR_NOGPU 5    /* no usable device                             */

/* ---- lifetime, errors ------------------------------------------------------
 * Replaces HipSetModuleImage / HipFinit (HipGpuUtils.cpp:39-47,154-159): the
 * kernels are linked into this library, there is no module image to load. */
int comet_hip_init(int device);
int comet_hip_finalize(void);
const char *comet_hip_last_error(void);
int comet_hip_device_name(char *buf, int64_t cap);

/* ---- raw device memory -----------------------------------------------------
 * Replaces HipMalloc{F64,F32,I64,I32} (HipGpuUtils.cpp:49-71), HipFree (:73-78)
 * and HipMemcpy* (:80-124; direction 0 = host to device, 1 = device to host). */
int64_t comet_hip_malloc(int64_t bytes);            /* 0 on failure */
int comet_hip_free(int64_t dptr);
int comet_hip_memcpy(int64_t dptr, void *host, int64_t bytes, int64_t direction);
int comet_hip_memset(int64_t dptr, int byte_value, int64_t bytes);
int comet_hip_sync(void);
/* A stream of the caller's own, as an integer (a hipStream_t, default
 * priority), for the entry points that take one; 0 on failure.  sync with 0
 * waits for the library's stream.  No counterpart in the reference, whose
 * runtime only knows the NULL stream (HipGpuUtils.cpp:21). */
int64_t comet_hip_stream_create(void);
int comet_hip_stream_sync(int64_t stream);
int comet_hip_stream_destroy(int64_t stream);
int64_t HipMallocF64(int64_t n);
int64_t HipMallocI64(int64_t n);
int64_t HipMallocI32(int64_t n);
void HipFree(int64_t dptr);
void HipMemcpyF64(int64_t dptr, void *ptr, void *aligned, int64_t offset, int64_t size, int64_t stride, int64_t dir);
void HipMemcpyI64(int64_t dptr, void *ptr, void *aligned, int64_t offset, int64_t size, int64_t stride, int64_t dir);
void HipMemcpyI32(int64_t dptr, void *ptr, void *aligned, int64_t offset, int64_t size, int64_t stride, int64_t dir);
void HipMemcpyIndex(int64_t dptr, void *ptr, void *aligned, int64_t offset, int64_t size, int64_t stride, int64_t dir);

/* ---- device CSR matrices ---------------------------------------------------
 * Device-side counterpart of the reader's CSR output (two-call "sizes then
 * fill" protocol of read_input_sizes_2D_f64 / read_input_2D_f64,
 * lib/ExecutionEngine/SparseUtils.cpp:1632-1811,1814-2078): upload takes the
 * host arrays the lowered code already owns; dims + download give them back.
 * Returns a handle (> 0) or 0 on failure.
 * Precondition, checked on the host before anything is copied: pos starts at 0,
 * never decreases and ends at nnz; every column lies in [0, ncols) and the
 * columns of a row do not decrease (what the reference's reader produces,
 * SparseUtils.cpp:421; the kernels bisect rows and index LDS by column).  The
 * reference's CPU loop nests would also accept rows in any column order; such
 * arrays are refused here - order them first with comet_hip_csr_from_coo_i64. */
int64_t comet_hip_csr_upload_i64(int64_t nrows, int64_t ncols, const int64_t *pos,
                                 const int64_t *crd, const double *val);
int64_t comet_hip_csr_upload_i32(int64_t nrows, int64_t ncols, const int32_t *pos,
                                 const int32_t *crd, const double *val);
/* Wrap device arrays the caller already filled (pos int64, crd int32, val f64);
 * the handle does not own them.  The kernels keep what they derive from a
 * matrix in its handle (re-ordered copies, block pointers, the transpose), so
 * after writing into wrapped arrays call comet_hip_csr_invalidate before the
 * handle is used again.  Both calls look at the arrays once on the device
 * (pos starts at 0, never decreases, ends at nnz; columns inside [0, ncols) and
 * not decreasing inside a row) and refuse anything else: wrap returns 0,
 * invalidate COMET_HIP_ERR_ARG - and the handle then refuses every product
 * (COMET_HIP_ERR_HANDLE) until a later invalidate passes or it is destroyed. */
int64_t comet_hip_csr_wrap(int64_t nrows, int64_t ncols, int64_t nnz,
                           int64_t pos_dptr, int64_t crd_dptr, int64_t val_dptr);
int comet_hip_csr_dims(int64_t csr, int64_t *nrows, int64_t *ncols, int64_t *nnz);
int comet_hip_csr_arrays(int64_t csr, int64_t *pos_dptr, int64_t *crd_dptr, int64_t *val_dptr);
int comet_hip_csr_download_i64(int64_t csr, int64_t *pos, int64_t *crd, double *val);
int comet_hip_csr_download_i32(int64_t csr, int32_t *pos, int32_t *crd, double *val);
int comet_hip_csr_invalidate(int64_t csr);
int comet_hip_csr_destroy(int64_t csr);

/* ---- SpMV  y[i] (+)= sum_p val[p] * x[crd[p]] ------------------------------
 * Replaces the loop nest of DenseParallelLoopInfo + SparseLoopInfo +
 * convertCompute (lib/Conversion/IndexTreeToSCF/IndexTreeToSCF.cpp:529-621,
 * 667-700,1247-1284).  accumulate != 0: y is added to, as the reference does;
 * accumulate == 0: y is overwritten (the result for a y the caller zero-filled,
 * without reading it).  x, y are device addresses of float64 vectors. */
int comet_hip_spmv_csr_f64(int64_t csr, int64_t x_dptr, int64_t y_dptr, int accumulate);

/* ---- SpMM  C[i,:] (+)= sum_p val[p] * B[crd[p],:] --------------------------
 * Same builders plus the dense inner loop (IndexTreeToSCF.cpp:476-489).
 * B is ncols x K with row stride ldb, C is nrows x K with row stride ldc
 * (elements).  accumulate as for SpMV.
 * Both products keep a plan in the handle (a re-ordered copy of parts of the
 * matrix) that costs tens of products to build: it is built when a handle is
 * multiplied for the second time, the first product runs without it.
 * Rounding: a row that lies inside one 256-nonzero chunk is summed in nonzero
 * order with separate multiply and add, bit for bit as the reference's nest
 * (IndexTreeToSCF.cpp:203-205); a row cut by a chunk boundary adds its pieces
 * in chunk order; the long rows a plan takes out (128 nonzeros and more) are
 * summed with fused multiply-adds from sixteen partial sums, so they agree
 * with the reference to rounding (1e-12 * sum |a||b|), never bitwise. */
int comet_hip_spmm_csr_f64(int64_t csr, int64_t K, int64_t b_dptr, int64_t ldb,
                           int64_t c_dptr, int64_t ldc, int accumulate);

/* The same product for callers that cannot allocate device memory (code under
 * HIP graph capture, serving loops and harnesses that forbid hipMalloc).  It has
 * no counterpart in the reference.  Nothing is allocated or freed: the scratch
 * of its kernels (chunk table and carry slots) is an 8 MiB array in the
 * library's image, one copy per device.  Limits: comet_hip_init must have run;
 * ceil(K/64) * ceil(nnz/256) <= 8192 (nnz <= 2,097,152 at K <= 64), larger
 * products return COMET_HIP_ERR_SIZE.  Rows are summed exactly as
 * comet_hip_spmm_csr_f64 sums them for a matrix below its long-row threshold.
 * All calls on one device share the array: calls that overlap in time race.
 * on_stream: the hipStream_t (as an integer) the kernels are launched on, so that
 * a caller that captures a graph or keeps a stream of its own gets them there,
 * ordered with its other work; 0 = the library's stream, as everywhere else. */
int comet_hip_spmm_csr_f64_noalloc(int64_t csr, int64_t K, int64_t b_dptr, int64_t ldb,
                                   int64_t c_dptr, int64_t ldc, int accumulate, int64_t on_stream);

/* ---- SpGEMM  C = A * B, CSR x CSR -> CSR, optional structural mask ---------
 * Symbolic phase: per-row count of distinct output columns and the row
 * pointer, replacing the mark-array nest of
 * lib/Dialect/IndexTree/Transforms/SymbolicCompute.cpp:215-339 as lowered by
 * lib/Conversion/IndexTreeToSCF/SymbolicDomainConversion.cpp:81-340.
 * Numeric phase: Gustavson accumulation and sorted row output, replacing the
 * workspace nest of lib/Dialect/IndexTree/Transforms/WorkspaceTransforms.cpp:
 * 97-276 as lowered by
 * lib/Conversion/TensorAlgebraToSCF/SparseTensorConversionPass.cpp:595-638,
 * 982-1159,261-327 (including its comet_sort call,
 * lib/ExecutionEngine/SparseUtils.cpp:2600-2626).
 * mask = 0 for none, else a CSR handle whose pattern restricts the output
 * (C[i,j] exists only where mask[i,j] is stored): MaskedDomainOp,
 * lib/Dialect/IndexTree/Transforms/IterationDomainInference.cpp:183-196,
 * lib/Conversion/IndexTreeToSCF/IndexTreeToSCF.cpp:1083-1148,1327-1448.
 * The output keeps every structurally reachable entry, also when its value
 * cancels to 0, with columns ascending per row. */
/* pos_dptr: device int64[nrows(A)+1], filled; *nnz_out = pos[nrows]. */
int comet_hip_spgemm_csr_symbolic(int64_t a, int64_t b, int64_t mask,
                                  int64_t pos_dptr, int64_t *nnz_out);
/* Rows [row_begin,row_end) of C into crd_dptr (int32) / val_dptr (float64),
 * written at offset pos[r] - pos[row_begin]; pos_dptr from the symbolic call. */
int comet_hip_spgemm_csr_numeric(int64_t a, int64_t b, int64_t mask, int64_t pos_dptr,
                                 int64_t row_begin, int64_t row_end,
                                 int64_t crd_dptr, int64_t val_dptr);
/* Both phases; returns a new CSR handle that owns its arrays (0 on failure). */
int64_t comet_hip_spgemm_csr(int64_t a, int64_t b, int64_t mask);

/* ---- SpGEMM over a semiring  C[a,c] = A[a,b] @(reduce, mult) B[b,c] ---------
 * The semiring forms of test/integration/semiring/mm_Semiring*_CSRxCSR_oCSR.ta
 * (frontends/comet_dsl/mlir/MLIRGen.cpp:101-147 for the names the DSL emits).
 * Per product e = mult(A[i,k], B[k,j]); C[i,j] = reduce over the products,
 * starting from the value the reference's workspace extract returns for an
 * untouched column: +inf for min, 0 otherwise - so max never returns less
 * than 0 (lib/Conversion/IndexTreeToSCF/IndexTreeToSCF.cpp:198-360,1190-1219,
 * 1249-1284).  "any" keeps the product a sequential traversal reaches last
 * (IndexTreeToSCF.cpp:346-349).  The structure of C does not depend on the
 * semiring, so the symbolic call above serves every one of them.  min, max
 * and any are independent of the order of evaluation and reproduce the
 * reference bit for bit (up to the sign of a zero); plus rounds like
 * comet_hip_spgemm_csr_numeric.  (COMET_SR_PLUS, COMET_OP_TIMES) is that
 * routine itself. */
enum { COMET_SR_PLUS = 0, COMET_SR_MIN = 1, COMET_SR_MAX = 2, COMET_SR_ANY = 3 };
enum { COMET_OP_TIMES = 0, COMET_OP_FIRST = 1, COMET_OP_SECOND = 2, COMET_OP_PAIR = 3, COMET_OP_PLUS = 4,
       COMET_OP_MINUS = 5, COMET_OP_MIN = 6, COMET_OP_MAX = 7, COMET_OP_DIV = 8 };
int comet_hip_spgemm_csr_numeric_semiring(int64_t a, int64_t b, int64_t mask, int64_t pos_dptr,
                                          int64_t row_begin, int64_t row_end,
                                          int64_t crd_dptr, int64_t val_dptr,
                                          int reduce_op, int mult_op);
int64_t comet_hip_spgemm_csr_semiring(int64_t a, int64_t b, int64_t mask, int reduce_op, int mult_op);

/* ---- dense operand on the left, and CSR .* Dense ------------------------------
 * y[j] (+)= sum_i x[i]*B[i,j] (test/integration/ops/mult_DenseVecxCSR.ta) and
 * C[a,c] (+)= sum_b A[a,b]*B[b,c], A: M x nrows(B) row-major with leading
 * dimension lda, C: M x ncols(B) (mult_DenseMatxCSR.ta); same index-tree lowering
 * as SpMV/SpMM with the sparse operand second.  An output element receives its
 * products in ascending order of the contracted index, as in the reference. */
int comet_hip_vecmat_csr_f64(int64_t csr, int64_t x_dptr, int64_t y_dptr, int accumulate);
int comet_hip_densemat_csr_f64(int64_t csr, int64_t M, int64_t a_dptr, int64_t lda,
                               int64_t c_dptr, int64_t ldc, int accumulate);
/* C = A (op) D elementwise for A in CSR and D dense (row-major, leading dimension
 * ldd); op is a COMET_OP_* code: COMET_OP_TIMES is the `.*` of the language,
 * the others its monoid forms `A @(+) D`, `@(-)`, `@(min)`, ...
 * (test/integration/semiring/eltwise_monoid*_COOxDense_oCOO.ta; lowering as
 * "noop_<op>", frontends/comet_dsl/mlir/MLIRGen.cpp:960-990).  A's value is the
 * left operand; for the source order D (op) A of a commutative op pass the same
 * call.  Result: a new CSR with A's structure (eltwise_mult_CSRxDense_oCSR.ta),
 * or written into a dense C at A's stored positions, every other element of C
 * left as it is (eltwise_mult_CSRxDense_oDense.ta, eltwise_mult_DensexCSR_oDense.ta). */
int64_t comet_hip_eltwise_csr_dense_csr(int64_t a, int64_t d_dptr, int64_t ldd, int op);
int comet_hip_eltwise_csr_dense_dense(int64_t a, int64_t d_dptr, int64_t ldd,
                                      int64_t c_dptr, int64_t ldc, int op);
/* c[i] = a[i] (op) b[i] over n dense elements
 * (eltwise_monoid{Plus,Minus,Min,Times}_DensexDense_oDense.ta). */
int comet_hip_eltwise_dense_f64(int64_t n, int64_t a_dptr, int64_t b_dptr, int64_t c_dptr, int op);

/* Sampled dense-dense matrix product, A = B .* (C x D): B is CSR (nrows x ncols), C is nrows x K (leading
 * dimension ldc), D is K x ncols (ldd), all fp64 on the device.  Returns a new CSR handle with B's structure
 * and val[p] * sum_k C[i,k] * D[k,j] for the stored entry p = (i, j), the sum unfused and in ascending k, as
 * the reference's loops compute it whether T = C x D is materialised or fused away (--opt-fusion,
 * lib/Dialect/IndexTree/Transforms/KernelFusion.cpp:1049-1220; test/integration/kernels/sddmm.ta:27-28).
 * The dense product is never formed.  0 on failure. */
int64_t comet_hip_sddmm_csr_f64(int64_t b, int64_t K, int64_t c_dptr, int64_t ldc, int64_t d_dptr, int64_t ldd);
/* The same values written to a device array of nnz(B) doubles the caller owns (A shares B's pos and crd, which
 * is how the lowered code holds the output of an elementwise operation: SparseTensorConversionPass.cpp:1281-1333
 * gives every sparse tensor its own value array).  Nothing is allocated for the result. */
int comet_hip_sddmm_csr_values_f64(int64_t b, int64_t K, int64_t c_dptr, int64_t ldc, int64_t d_dptr,
                                   int64_t ldd, int64_t out_val_dptr);

/* ---- input side: MatrixMarket files, read modes, the file-id protocol ---------
 * Read modes of comet_read(id, mode): lib/ExecutionEngine/SparseUtils.cpp:40-64.
 * Storage format codes per dimension: include/comet/ExecutionEngine/
 * RunnerUtils.h:71-77. */
enum { COMET_READ_DEFAULT = 1, COMET_READ_LOWER_TRI_STRICT = 2, COMET_READ_LOWER_TRI = 3,
       COMET_READ_UPPER_TRI_STRICT = 4, COMET_READ_UPPER_TRI = 5 };
enum { COMET_FMT_DENSE = 0, COMET_FMT_COMPRESSED_UNIQUE = 1, COMET_FMT_COMPRESSED_NONUNIQUE = 2,
       COMET_FMT_SINGLETON = 3 };
/* Parse a MatrixMarket file (coordinate or array; general, symmetric or skew;
 * a missing value reads as 1.0) on the host, then order, filter by read mode
 * and build CSR on the GPU: CooMatrix::InitMarket + CsrMatrix::Init,
 * SparseUtils.cpp:145-356,404-533.  Duplicates are kept in file order.
 * Returns a CSR handle (0 on failure). */
int64_t comet_hip_mtx_read_csr(const char *path, int read_mode);
/* The reader's two calls, SparseUtils.cpp:1632-1810 (read_input_sizes_2D_f64)
 * and :1814-2050 (read_input_2D_f64_i64), with their argument lists: file_id
 * 0..9998 names the environment variable SPARSE_FILE_NAME<id>, 9999
 * SPARSE_FILE_NAME (:1444-1466); every (rank, descriptor) pair is an unranked
 * memref whose descriptor is a rank-1 strided memref of int64 (float64 for
 * Aval).  Layouts read: CSR (Dense, Compressed_unique), COO
 * (Compressed_nonunique, singleton), DCSR (Compressed_unique,
 * Compressed_unique); any other prints a message and exits, like every failure
 * of these two calls in the reference.  sizes[0..10] as in the reference;
 * arrays a layout does not use get -1 in their first element.  The sizes call
 * builds the device CSR and keeps it for the read call that follows. */
void comet_hip_read_input_sizes_2D_f64(int32_t file_id, int32_t a1format, int32_t a1_tile_format,
                                       int32_t a2format, int32_t a2_tile_format,
                                       int sizes_rank, void *sizes_desc, int32_t read_mode);
void comet_hip_read_input_2D_f64_i64(int32_t file_id, int32_t a1format, int32_t a1_tile_format,
                                     int32_t a2format, int32_t a2_tile_format,
                                     int a1pos_rank, void *a1pos_desc, int a1crd_rank, void *a1crd_desc,
                                     int a1tile_pos_rank, void *a1tile_pos_desc,
                                     int a1tile_crd_rank, void *a1tile_crd_desc,
                                     int a2pos_rank, void *a2pos_desc, int a2crd_rank, void *a2crd_desc,
                                     int a2tile_pos_rank, void *a2tile_pos_desc,
                                     int a2tile_crd_rank, void *a2tile_crd_desc,
                                     int aval_rank, void *aval_desc, int32_t read_mode);
/* The reader for lowered code built with --target=GPU, whose index memrefs
 * hold int32 (frontends/comet_dsl/comet.cpp:817-823): read_input_2D_f64_i32,
 * SparseUtils.cpp:2403-2425.  Same protocol; the sizes call is shared (sizes are
 * `index` values for either width). */
void comet_hip_read_input_2D_f64_i32(int32_t file_id, int32_t a1format, int32_t a1_tile_format,
                                     int32_t a2format, int32_t a2_tile_format,
                                     int a1pos_rank, void *a1pos_desc, int a1crd_rank, void *a1crd_desc,
                                     int a1tile_pos_rank, void *a1tile_pos_desc,
                                     int a1tile_crd_rank, void *a1tile_crd_desc,
                                     int a2pos_rank, void *a2pos_desc, int a2crd_rank, void *a2crd_desc,
                                     int a2tile_pos_rank, void *a2tile_pos_desc,
                                     int a2tile_crd_rank, void *a2tile_crd_desc,
                                     int aval_rank, void *aval_desc, int32_t read_mode);
/* The three calls under the names lowered code already calls
 * (lib/ExecutionEngine/SparseUtils.cpp:2562-2568, 2403-2425, 2427-2450): with this
 * library in -shared-libs in place of libcomet_runner_utils, `ta.read` resolves
 * without a compiler change.  Same argument lists and behaviour as above. */
void read_input_sizes_2D_f64(int32_t file_id, int32_t a1format, int32_t a1_tile_format,
                             int32_t a2format, int32_t a2_tile_format,
                             int sizes_rank, void *sizes_desc, int32_t read_mode);
void read_input_2D_f64_i64(int32_t file_id, int32_t a1format, int32_t a1_tile_format,
                           int32_t a2format, int32_t a2_tile_format,
                           int a1pos_rank, void *a1pos_desc, int a1crd_rank, void *a1crd_desc,
                           int a1tile_pos_rank, void *a1tile_pos_desc,
                           int a1tile_crd_rank, void *a1tile_crd_desc,
                           int a2pos_rank, void *a2pos_desc, int a2crd_rank, void *a2crd_desc,
                           int a2tile_pos_rank, void *a2tile_pos_desc,
                           int a2tile_crd_rank, void *a2tile_crd_desc,
                           int aval_rank, void *aval_desc, int32_t read_mode);
void read_input_2D_f64_i32(int32_t file_id, int32_t a1format, int32_t a1_tile_format,
                           int32_t a2format, int32_t a2_tile_format,
                           int a1pos_rank, void *a1pos_desc, int a1crd_rank, void *a1crd_desc,
                           int a1tile_pos_rank, void *a1tile_pos_desc,
                           int a1tile_crd_rank, void *a1tile_crd_desc,
                           int a2pos_rank, void *a2pos_desc, int a2crd_rank, void *a2crd_desc,
                           int a2tile_pos_rank, void *a2tile_pos_desc,
                           int a2tile_crd_rank, void *a2tile_crd_desc,
                           int aval_rank, void *aval_desc, int32_t read_mode);
/* The same read for lowered code that keeps tensors on the device: the CSR
 * handle itself (0 on failure), no host arrays.  Consumes what a preceding
 * sizes call for the same id and mode built, or reads the file now. */
int64_t comet_hip_read_input_2D_handle(int32_t file_id, int32_t read_mode);

/* ---- the other matrix layouts of the reference's SpMV/SpMM tests ------------
 * COO = {Compressed_nonunique, singleton}: A1pos = [0, nnz], A1crd = rows,
 * A2crd = columns (SparseUtils.cpp:1855-1896); DCSR = {Compressed_unique,
 * Compressed_unique}: A1pos = [0, stored rows], A1crd = ids of the rows that
 * store anything, A2pos/A2crd/Aval as in CSR over those rows (:669-735).
 * test/integration/ops/mult_spm{v,m}_{COO,DCSR}xDense.ta run on the CSR
 * kernels after one of these conversions.  Tuples may come in any order
 * (ordered on the GPU, ties keep input order); read_mode filters as above. */
int64_t comet_hip_csr_from_coo_i64(int64_t nrows, int64_t ncols, int64_t nnz, const int64_t *row,
                                   const int64_t *col, const double *val, int read_mode);
/* The same for tuples that already sit in HBM: int32 rows and columns, float64
 * values; a tuple outside the matrix is refused (checked on the device). */
int64_t comet_hip_csr_from_coo_device(int64_t nrows, int64_t ncols, int64_t nnz, int64_t row_dptr,
                                      int64_t col_dptr, int64_t val_dptr, int read_mode);
int64_t comet_hip_csr_from_dcsr_i64(int64_t nrows, int64_t ncols, int64_t nrows_stored,
                                    const int64_t *a1crd, const int64_t *a2pos,
                                    const int64_t *a2crd, const double *aval);
/* Host arrays of nnz entries each. */
int comet_hip_csr_to_coo_i64(int64_t csr, int64_t *row, int64_t *col, double *val);
/* *nrows_stored is always written; with all four arrays null this is the size
 * query (a1crd: stored, a2pos: stored + 1, a2crd/aval: nnz). */
int comet_hip_csr_to_dcsr_i64(int64_t csr, int64_t *nrows_stored, int64_t *a1crd, int64_t *a2pos,
                              int64_t *a2crd, double *aval);
/* New handle holding the transpose, columns ascending per row (the CSR -> CSC
 * reordering of lib/ExecutionEngine/TransposeUtils.cpp done as one device sort). */
int64_t comet_hip_csr_transpose(int64_t csr);

/* ---- masked SpGEMM + SUM in one pass (triangle counting) -------------------
 * *out = SUM(C) for C<L> = L * L, the two statements of
 * test/integration/kernels/triangleCount_SandiaLL_wMasking.ta:18-39, i.e. the
 * masked numeric phase followed by ReduceOpLowering
 * (lib/Conversion/TensorAlgebraToSCF/TensorAlgebraToSCF.cpp:417-529), without
 * materialising C.  a, b, mask may all be the same handle.
 * When every stored value of b is one number (a pattern matrix, looked at once per
 * handle), the kernels count per row of b how many of its columns the mask row
 * holds and add count * (a's entry * that number): sums of whole numbers, such as
 * a triangle count, are exact; other values agree with the product-by-product sum
 * to rounding.  COMET_HIP_MASKED_SUM_ONLY=workgroup|wavefront in the environment
 * sends every row through one of the two kernels (a diagnostic: the tests use it). */
int comet_hip_spgemm_masked_sum(int64_t a, int64_t b, int64_t mask, double *out);

/* ---- SUM over a device float64 array (ReduceOpLowering, as above) --------- */
int comet_hip_reduce_sum_f64(int64_t dptr, int64_t n, double *out);

/* ---- CSR .* CSR -> CSR (two-pointer intersection nest,
 * lib/Conversion/IndexTreeToSCF/IndexTreeToSCF.cpp:864-1053).  New handle. */
int64_t comet_hip_eltwise_mult_csr(int64_t a, int64_t b);

/* ---- dense tensor transpose, linalg.transpose semantics --------------------
 * out dim i = in dim perm[i] (how TCtoTTGTDyn.cpp:288-329 builds its
 * transposes); contiguous row-major float64; rank <= 8. */
int comet_hip_transpose_f64(int32_t rank, const int64_t *in_shape, const int32_t *perm,
                            int64_t in_dptr, int64_t out_dptr);

/* ---- row-major DGEMM  C[M,N] = beta*C + A[M,K] * B[K,N] --------------------
 * Replaces linalg.matmul lowered to loops (frontends/comet_dsl/comet.cpp:
 * 594-595) and the tiled BLIS micro-kernel path
 * (_mlir_ciface_linalg_matmul_viewsxs_viewsxs_viewsxs,
 * lib/ExecutionEngine/blis_interface.cpp:143-181). beta is 0 or 1. */
int comet_hip_dgemm_f64(int64_t M, int64_t N, int64_t K, int64_t a_dptr, int64_t b_dptr,
                        int64_t c_dptr, double beta);

/* ---- TTGT contraction ------------------------------------------------------
 * Plan: index classification, candidate enumeration, cost rule and selection
 * of include/comet/Dialect/Utils/Utils.h:586-946 and
 * lib/Dialect/TensorAlgebra/Transforms/TCtoTTGTDyn.cpp:240-272.
 * x_lab: label id of each dimension in storage order; extent[label] its size;
 * which = -1 selects by cost (first strict minimum), >= 0 forces a candidate
 * (--perm-num). */
typedef struct {
    int32_t rankA, rankB, rankC;
    int32_t a_idx[8], b_idx[8], c_idx[8];    /* label order after the transposes      */
    int32_t permA[8], permB[8], permC[8];    /* linalg.transpose permutations         */
    int32_t transA, transB, transC, swapAB;  /* which transposes run; operand swap    */
    int64_t M, N, K;
    double cost;
    int32_t candidate, ncandidates;
} comet_ttgt_plan;
int comet_hip_ttgt_plan(int32_t rankA, const int32_t *a_lab, int32_t rankB, const int32_t *b_lab,
                        int32_t rankC, const int32_t *c_lab, const int64_t *extent, int32_t which,
                        comet_ttgt_plan *plan);
/* Execute: transposes -> DGEMM -> inverse transpose (TCtoTTGTDyn.cpp:280-672).
 * a/b/c are device float64 tensors in their declared layouts; workspace for the
 * transposed copies is owned and cached by the library. */
int comet_hip_ttgt_contract(const comet_ttgt_plan *plan, const int64_t *a_shape,
                            const int64_t *b_shape, const int64_t *c_shape,
                            int64_t a_dptr, int64_t b_dptr, int64_t c_dptr, double beta);

/* ---- timing ----------------------------------------------------------------
 * HIP events on the library's stream (the reference's getTime /
 * printElapsedTime, lib/ExecutionEngine/StatUtils.cpp:42-59, measure host wall
 * clock and cannot see asynchronous kernels).
 * timer_start/stop bracket a region; kernel profiling, when enabled, records an
 * event pair around every kernel launch and sums them per kernel name. */
int comet_hip_timer_start(void);
int comet_hip_timer_stop(double *ms);
int comet_hip_profile_enable(int on);
int comet_hip_profile_reset(void);
/* name == NULL: number of distinct kernel names recorded so far. */
int comet_hip_profile_query(const char *name, int64_t *launches, double *total_ms);
int comet_hip_profile_name(int32_t index, char *buf, int64_t cap);
/* ---- diagnostics: yardsticks the measurements are set against -----------------
 * None of the functions from here to comet_hip_gather_rows_bench has a
 * counterpart in the reference and none is on the product path; they exist so
 * that a roofline fraction can be read against what the machine does on the
 * simplest kernel of the same kind. */
/* Plain device-to-device copy kernel, 8 bytes per lane (used to calibrate
 * hardware counters). */
int comet_hip_copy_f64(int64_t dst_dptr, int64_t src_dptr, int64_t n);
/* Streaming kernels with 16 bytes per lane over n doubles (n even, pointers
 * 16-byte aligned).  mode 0: copy with ordinary loads and stores; 1: copy with
 * non-temporal loads and stores; 2: read only (src; every lane sums what it
 * reads); 3: write only (dst).  workgroups_per_cu: 256-lane workgroups per CU in
 * the grid, 0 = 8. */
int comet_hip_stream_bench(int mode, int64_t dst_dptr, int64_t src_dptr, int64_t n, int workgroups_per_cu);
/* Free and total device memory (hipMemGetInfo): lets a caller see what a first
 * call kept (plans cached in a handle, workspaces). */
int comet_hip_mem_info(int64_t *free_bytes, int64_t *total_bytes);
/* Two more diagnostics.  mfma_f64_peak: TFLOP/s of back-to-back v_mfma_f64_16x16x4_f64
 * on registers (`iters` x 16 per wavefront, 8 wavefronts per CU), the rate the
 * TTGT GEMM is compared with.  gather_rows_bench: every wavefront fetches
 * per_wave rows of 64 doubles named by idx (int32, one list per wavefront, 16
 * wavefronts per workgroup) from `table`, half a wavefront per row and 16 bytes
 * per lane as the SpMM sweep does, and sums them into out (workgroups x 1024
 * doubles): the rate at which the CUs can take rows out of the L2. */
int comet_hip_mfma_f64_peak(int64_t iters, double *tflops);
/* Diagnostic: the word offset at which the fp64 sums of the masked-product
 * kernel begin in its LDS for a bitmap of `words` 32-bit words; always even (an
 * odd offset would misalign its 64-bit LDS atomics).  Runs on the host. */
int comet_hip_debug_dot_table_words(int words);
/* Diagnostic: vector registers per lane of the two kernels of the pattern-matrix
 * masked sum (comet_hip_spgemm_masked_sum) in the loaded code object.  They share
 * the CUs, and do so only while four wavefronts of the first and one of the second
 * fit a SIMD's 512 registers. */
int comet_hip_debug_masked_sum_registers(int *workgroup_kernel, int *wavefront_kernel);
int comet_hip_gather_rows_bench(int64_t workgroups, int64_t per_wave, int64_t idx_dptr,
                                int64_t table_dptr, int64_t table_rows, int64_t out_dptr);

/* ---- memref-descriptor forms ----------------------------------------------
 * What `func.call` sites in lowered code bind to (llvm.emit_c_interface):
 * pointers to StridedMemRefType<T,N> {T* allocated; T* aligned; int64 offset;
 * int64 sizes[N]; int64 strides[N]} holding HOST data, exactly as the
 * reference's other runtime calls receive them
 * (lib/ExecutionEngine/StatUtils.cpp:89-113, blis_interface.cpp:143-146).
 * They upload, run the kernel, and copy the result back.  The CSR operands
 * must satisfy the precondition stated at comet_hip_csr_upload_* (columns of a
 * row not decreasing): an operand that does not ends the program with a message,
 * as every failure of these forms does. */
typedef struct { void *allocated; void *aligned; int64_t offset; int64_t sizes[1]; int64_t strides[1]; } comet_memref_1d;
typedef struct { void *allocated; void *aligned; int64_t offset; int64_t sizes[2]; int64_t strides[2]; } comet_memref_2d;

void _mlir_ciface_comet_hip_spmv_csr_f64_i64(comet_memref_1d *pos, comet_memref_1d *crd, comet_memref_1d *val,
                                             comet_memref_1d *x, comet_memref_1d *y);
void _mlir_ciface_comet_hip_spmm_csr_f64_i64(comet_memref_1d *pos, comet_memref_1d *crd, comet_memref_1d *val,
                                             comet_memref_2d *B, comet_memref_2d *C);
/* SpGEMM in the reader's two-call style: sizes first (nnz of C into
 * sizes[0]; keeps the device result cached), then fill. */
void _mlir_ciface_comet_hip_spgemm_csr_sizes_f64_i64(int64_t nrowsA, int64_t ncolsB,
        comet_memref_1d *Apos, comet_memref_1d *Acrd, comet_memref_1d *Aval,
        comet_memref_1d *Bpos, comet_memref_1d *Bcrd, comet_memref_1d *Bval,
        comet_memref_1d *Mpos, comet_memref_1d *Mcrd, comet_memref_1d *sizes);
void _mlir_ciface_comet_hip_spgemm_csr_fill_f64_i64(comet_memref_1d *Cpos, comet_memref_1d *Ccrd,
                                                    comet_memref_1d *Cval);
double _mlir_ciface_comet_hip_tricount_f64_i64(int64_t ncols, comet_memref_1d *pos, comet_memref_1d *crd,
                                               comet_memref_1d *val);

/* The same five entry points for index memrefs of int32 (pos, crd and the mask's
 * arrays; `sizes` stays int64): what lowered code built with --target=GPU passes
 * (frontends/comet_dsl/comet.cpp:817-823). */
void _mlir_ciface_comet_hip_spmv_csr_f64_i32(comet_memref_1d *pos, comet_memref_1d *crd, comet_memref_1d *val,
                                             comet_memref_1d *x, comet_memref_1d *y);
void _mlir_ciface_comet_hip_spmm_csr_f64_i32(comet_memref_1d *pos, comet_memref_1d *crd, comet_memref_1d *val,
                                             comet_memref_2d *B, comet_memref_2d *C);
void _mlir_ciface_comet_hip_spgemm_csr_sizes_f64_i32(int64_t nrowsA, int64_t ncolsB,
        comet_memref_1d *Apos, comet_memref_1d *Acrd, comet_memref_1d *Aval,
        comet_memref_1d *Bpos, comet_memref_1d *Bcrd, comet_memref_1d *Bval,
        comet_memref_1d *Mpos, comet_memref_1d *Mcrd, comet_memref_1d *sizes);
void _mlir_ciface_comet_hip_spgemm_csr_fill_f64_i32(comet_memref_1d *Cpos, comet_memref_1d *Ccrd,
                                                    comet_memref_1d *Cval);
double _mlir_ciface_comet_hip_tricount_f64_i32(int64_t ncols, comet_memref_1d *pos, comet_memref_1d *crd,
                                               comet_memref_1d *val);

/* SpGEMM over a semiring through the same pair of calls: the operator codes of
 * comet_hip_spgemm_csr_semiring after the sizes memref
 * (lib/Conversion/IndexTreeToSCF/IndexTreeToSCF.cpp:198-360;
 * test/integration/semiring/mm_Semiring*_CSRxCSR_oCSR.ta).  The fill call is the
 * plain one under a second name. */
void _mlir_ciface_comet_hip_spgemm_csr_sizes_semiring_f64_i64(int64_t nrowsA, int64_t ncolsB,
        comet_memref_1d *Apos, comet_memref_1d *Acrd, comet_memref_1d *Aval,
        comet_memref_1d *Bpos, comet_memref_1d *Bcrd, comet_memref_1d *Bval,
        comet_memref_1d *Mpos, comet_memref_1d *Mcrd, comet_memref_1d *sizes,
        int32_t reduce_op, int32_t mult_op);
void _mlir_ciface_comet_hip_spgemm_csr_fill_semiring_f64_i64(comet_memref_1d *Cpos, comet_memref_1d *Ccrd,
                                                             comet_memref_1d *Cval);
void _mlir_ciface_comet_hip_spgemm_csr_sizes_semiring_f64_i32(int64_t nrowsA, int64_t ncolsB,
        comet_memref_1d *Apos, comet_memref_1d *Acrd, comet_memref_1d *Aval,
        comet_memref_1d *Bpos, comet_memref_1d *Bcrd, comet_memref_1d *Bval,
        comet_memref_1d *Mpos, comet_memref_1d *Mcrd, comet_memref_1d *sizes,
        int32_t reduce_op, int32_t mult_op);
void _mlir_ciface_comet_hip_spgemm_csr_fill_semiring_f64_i32(comet_memref_1d *Cpos, comet_memref_1d *Ccrd,
                                                             comet_memref_1d *Cval);

/* Dense contraction on host memrefs: upload -> plan -> transposes -> GEMM ->
 * download in one call, in place of the transpose / collapse / matmul / expand /
 * transpose chain the reference emits
 * (lib/Dialect/TensorAlgebra/Transforms/TCtoTTGTDyn.cpp:288-672).  A, B, C are
 * unranked memrefs (rank, pointer to StridedMemRefType<double, rank>), rank 1..8,
 * contiguous row-major; x_lab holds one `index` per dimension, the same number
 * for the same index label (C[a,b,c,d] = A[a,e,b,f] * B[d,f,c,e]: 0,4,1,5 /
 * 3,5,2,4 / 0,1,2,3); beta 0 overwrites C, 1 adds to it. */
void _mlir_ciface_comet_hip_ttgt_contract_f64(int64_t rankA, void *A, int64_t rankB, void *B,
                                              int64_t rankC, void *C, comet_memref_1d *a_lab,
                                              comet_memref_1d *b_lab, comet_memref_1d *c_lab, double beta);
/* The reference's own name for the matrix product its TTGT lowering ends in
 * under -opt-matmul-mkernel (lib/ExecutionEngine/blis_interface.cpp:143-181):
 * C = alpha * A * B + beta * C on strided 2-D views of host memory.  mr and nr
 * (the micro-kernel's tile) are ignored: the whole product runs on the device. */
void _mlir_ciface_linalg_matmul_viewsxs_viewsxs_viewsxs(comet_memref_2d *A, comet_memref_2d *B,
                                                        comet_memref_2d *C, int mr, int nr,
                                                        double alpha, double beta);

/* ---- host utilities of the reference's runtime ----------------------------
 * The names and argument lists lowered programs already call
 * (lib/ExecutionEngine/StatUtils.cpp:42-59,109-137, SparseUtils.cpp:2610-2626), so that this library can
 * stand alone behind -shared-libs.  An unranked memref is (rank, pointer to StridedMemRefType<T, rank>).
 * Printing follows include/comet/ExecutionEngine/RunnerUtils.h:232-266 ("data = ", line break, every element
 * and a comma, line break; nothing for an empty tensor).  getTime drains the device first. */
void comet_print_memref_f64(int64_t rank, void *desc);
void comet_print_memref_f32(int64_t rank, void *desc);
void comet_print_memref_i64(int64_t rank, void *desc);
void comet_print_memref_i32(int64_t rank, void *desc);
void comet_print_memref_index(int64_t rank, void *desc);
void comet_sort_index(int64_t rank, void *desc, int64_t first, int64_t last);
void comet_sort64(int64_t rank, void *desc, int64_t first, int64_t last);
void comet_sort32(int64_t rank, void *desc, int64_t first, int64_t last);
double getTime(void);
void printElapsedTime(double stime, double etime);

#ifdef __cplusplus
}
#endif
#endif /* COMET_HIP_RT_H */
