// TTGT dense contraction for gfx950: the permutation plan, tensor transposes
// staged through LDS, and an fp64 MFMA GEMM.
//
// Plan = index classification, candidate enumeration, cost rule and selection
// of include/comet/Dialect/Utils/Utils.h:586-946 and
// lib/Dialect/TensorAlgebra/Transforms/TCtoTTGTDyn.cpp:240-272 in pnnl/COMET.
// Execution = the transpose -> collapse -> matmul -> expand -> transpose chain
// of TCtoTTGTDyn.cpp:280-672, with the matmul
// (linalg.matmul -> loops, frontends/comet_dsl/comet.cpp:594-595, or the BLIS
// micro-kernel of lib/ExecutionEngine/blis_interface.cpp:143-181) replaced by
// v_mfma_f64_16x16x4_f64 tiles.
#include <algorithm>
#include <cstring>

#include "common.h"

namespace comet {

// ============================================================================
// Transposes.  out dim i = in dim perm[i]; both tensors contiguous row-major.
// Dimensions that stay adjacent are merged first.  If the innermost dimension
// is kept, rows are copied (coalesced on both sides).  Otherwise the innermost
// input dimension (b) and the innermost output dimension (a) form 2-D tiles
// that go through LDS, so that reads run along b and writes run along a.
// ============================================================================
constexpr int TR_MAXRANK = 8;
constexpr int TR_TILE = 32;

struct TrDims {
    int rank;
    int64_t out_shape[TR_MAXRANK];
    int64_t src_stride[TR_MAXRANK];   // input stride of output dim i
    int64_t out_stride[TR_MAXRANK];
};

__global__ __launch_bounds__(256) void transpose_rows_kernel(TrDims d, int64_t total, const double *__restrict__ in,
                                                             double *__restrict__ out)
{
    int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; o < total; o += step) {
        int64_t rem = o, src = 0;
        for (int i = d.rank - 1; i >= 0; --i) {
            const int64_t c = rem % d.out_shape[i];
            rem /= d.out_shape[i];
            src += c * d.src_stride[i];
        }
        out[o] = in[src];
    }
}

// Tile over (a = output-innermost dim, b = input-innermost dim).  Batch index =
// all other output dims, flattened in output order.
struct TrTile {
    int nbatch_dims;
    int64_t batch_shape[TR_MAXRANK];
    int64_t batch_src_stride[TR_MAXRANK];
    int64_t batch_out_stride[TR_MAXRANK];
    int64_t na, nb;                // extents of a and b
    int64_t a_src_stride;          // input stride of a  (input stride of b is 1)
    int64_t b_out_stride;          // output stride of b (output stride of a is 1)
};

__global__ __launch_bounds__(256) void transpose_tile_kernel(TrTile d, const double *__restrict__ in,
                                                             double *__restrict__ out)
{
    __shared__ double tile[TR_TILE][TR_TILE + 1];
    int64_t rem = blockIdx.z;
    int64_t src = 0, dst = 0;
    for (int i = d.nbatch_dims - 1; i >= 0; --i) {
        const int64_t c = rem % d.batch_shape[i];
        rem /= d.batch_shape[i];
        src += c * d.batch_src_stride[i];
        dst += c * d.batch_out_stride[i];
    }
    const int64_t a0 = (int64_t)blockIdx.x * TR_TILE, b0 = (int64_t)blockIdx.y * TR_TILE;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;   // 32 x 8
    for (int r = ty; r < TR_TILE; r += 8) {
        const int64_t a = a0 + r, b = b0 + tx;
        if (a < d.na && b < d.nb)
            tile[r][tx] = in[src + a * d.a_src_stride + b];
    }
    __syncthreads();
    for (int r = ty; r < TR_TILE; r += 8) {
        const int64_t b = b0 + r, a = a0 + tx;
        if (a < d.na && b < d.nb)
            out[dst + b * d.b_out_stride + a] = tile[tx][r];
    }
}

static int transpose_device(int rank, const int64_t *in_shape, const int32_t *perm, const double *in, double *out)
{
    if (rank < 1 || rank > TR_MAXRANK)
        return set_error(COMET_HIP_ERR_ARG, "transpose rank %d outside [1,%d]", rank, TR_MAXRANK);
    bool seen[TR_MAXRANK] = {false};
    int64_t total = 1;
    for (int i = 0; i < rank; ++i) {
        if (perm[i] < 0 || perm[i] >= rank || seen[perm[i]])
            return set_error(COMET_HIP_ERR_ARG, "perm is not a permutation of 0..%d", rank - 1);
        seen[perm[i]] = true;
        if (in_shape[i] < 0)
            return set_error(COMET_HIP_ERR_ARG, "negative extent");
        total *= in_shape[i];
    }
    if (total == 0)
        return COMET_HIP_OK;
    int64_t in_stride[TR_MAXRANK];
    {
        int64_t s = 1;
        for (int i = rank - 1; i >= 0; --i) {
            in_stride[i] = s;
            s *= in_shape[i];
        }
    }
    // output dims with merging of runs that are adjacent in the input too; extent-1 dims dropped
    int n = 0;
    int64_t shp[TR_MAXRANK], sst[TR_MAXRANK];
    int last_in = -2;
    for (int i = 0; i < rank; ++i) {
        const int p = perm[i];
        if (in_shape[p] == 1)
            continue;
        if (n > 0 && p == last_in + 1) {
            shp[n - 1] *= in_shape[p];
            sst[n - 1] = in_stride[p];
        } else {
            shp[n] = in_shape[p];
            sst[n] = in_stride[p];
            ++n;
        }
        last_in = p;
    }
    if (n == 0) {   // single element
        COMET_HIPCHK(hipMemcpyAsync(out, in, sizeof(double), hipMemcpyDeviceToDevice, stream()));
        return COMET_HIP_OK;
    }
    int64_t ost[TR_MAXRANK];
    {
        int64_t s = 1;
        for (int i = n - 1; i >= 0; --i) {
            ost[i] = s;
            s *= shp[i];
        }
    }
    if (n == 1) {
        COMET_HIPCHK(hipMemcpyAsync(out, in, sizeof(double) * (size_t)total, hipMemcpyDeviceToDevice, stream()));
        return COMET_HIP_OK;
    }
    if (sst[n - 1] == 1) {   // innermost kept
        TrDims d;
        d.rank = n;
        for (int i = 0; i < n; ++i) {
            d.out_shape[i] = shp[i];
            d.src_stride[i] = sst[i];
            d.out_stride[i] = ost[i];
        }
        const unsigned blocks = (unsigned)std::min<int64_t>(ceil_div(total, 256), (int64_t)num_cus() * 64);
        KernelTimer t("transpose_rows_kernel");
        transpose_rows_kernel<<<dim3(blocks), dim3(256), 0, stream()>>>(d, total, in, out);
        COMET_HIPCHK(hipGetLastError());
        return COMET_HIP_OK;
    }
    // find the output dim that is innermost in the input
    int bdim = -1;
    for (int i = 0; i < n; ++i)
        if (sst[i] == 1)
            bdim = i;
    if (bdim < 0)
        return set_error(COMET_HIP_ERR_ARG, "internal: no unit-stride dimension");
    TrTile d;
    d.nbatch_dims = 0;
    int64_t nbatch = 1;
    for (int i = 0; i < n - 1; ++i) {
        if (i == bdim)
            continue;
        d.batch_shape[d.nbatch_dims] = shp[i];
        d.batch_src_stride[d.nbatch_dims] = sst[i];
        d.batch_out_stride[d.nbatch_dims] = ost[i];
        ++d.nbatch_dims;
        nbatch *= shp[i];
    }
    d.na = shp[n - 1];
    d.nb = shp[bdim];
    d.a_src_stride = sst[n - 1];
    d.b_out_stride = ost[bdim];
    const int64_t ga = ceil_div(d.na, TR_TILE), gb = ceil_div(d.nb, TR_TILE);
    if (gb > 65535 || nbatch > 65535) {
        // fall back to the gather kernel when the grid would not fit
        TrDims g;
        g.rank = n;
        for (int i = 0; i < n; ++i) {
            g.out_shape[i] = shp[i];
            g.src_stride[i] = sst[i];
            g.out_stride[i] = ost[i];
        }
        const unsigned blocks = (unsigned)std::min<int64_t>(ceil_div(total, 256), (int64_t)num_cus() * 64);
        KernelTimer t("transpose_rows_kernel");
        transpose_rows_kernel<<<dim3(blocks), dim3(256), 0, stream()>>>(g, total, in, out);
        COMET_HIPCHK(hipGetLastError());
        return COMET_HIP_OK;
    }
    KernelTimer t("transpose_tile_kernel");
    transpose_tile_kernel<<<dim3((unsigned)ga, (unsigned)gb, (unsigned)nbatch), dim3(256), 0, stream()>>>(d, in, out);
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}

// ============================================================================
// DGEMM, row-major, C[M,N] = beta*C + A[M,K]*B[K,N].
// Workgroup tile 128 x 128, four wavefronts in a 2 x 2 arrangement, each
// wavefront 64 x 64 as 4 x 4 MFMA tiles (16 accumulators of 4 doubles per
// lane).  K advances 16 at a time through double-buffered LDS: A is stored
// k-major (so a 16 x 4 operand is read with one ds_read_b64 per lane), B as in
// memory.  Operand layout of v_mfma_f64_16x16x4_f64: lane l supplies
// A[l%16][l/16] and B[l/16][l%16] and receives D[4*v + l/16][l%16], v = 0..3
// (measured on gfx950 with one-hot operands).
// ============================================================================
#ifndef COMET_GM_BK
#define COMET_GM_BK 16
#endif
#ifndef COMET_GM_PAD
#define COMET_GM_PAD 4
#endif
#ifndef COMET_GM_OCC
#define COMET_GM_OCC 2
#endif
// Measured on the 4096^3 product: 2 wavefronts per SIMD (register budget 256) lifts the kernel from 62 % to
// 90 % of the fp64 MFMA peak; a deeper K tile (32) does not fit two workgroups' LDS and falls back to 59 %.
constexpr int GM_BM = 128, GM_BN = 128, GM_BK = COMET_GM_BK;
constexpr int GM_LDA = GM_BM + COMET_GM_PAD;   // padded leading dimensions (doubles)
constexpr int GM_LDB = GM_BN + COMET_GM_PAD;
constexpr int GM_EA = GM_BM * GM_BK / 256;     // doubles each lane stages per tile of A (along k)
constexpr int GM_EB = GM_BK * GM_BN / 256;     // ... and of B (along n)

typedef double double4_t __attribute__((ext_vector_type(4)));

template <bool GUARD>
__global__ __launch_bounds__(256, COMET_GM_OCC) void dgemm_mfma_kernel(int64_t M, int64_t N, int64_t K,
                                                         const double *__restrict__ A,
                                                         const double *__restrict__ B, double *__restrict__ C,
                                                         int use_c)
{
    __shared__ double As[2][GM_BK][GM_LDA];
    __shared__ double Bs[2][GM_BK][GM_LDB];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    // neighbouring workgroups share a block row of A: walk N fastest inside groups of 8 block rows
    const int64_t bm = blockIdx.y, bn = blockIdx.x;
    const int64_t m0 = bm * GM_BM, n0 = bn * GM_BN;

    // global -> register staging: A tile 128 x BK (two lanes per row, GM_EA consecutive k each),
    // B tile BK x 128 (GM_EB consecutive columns per lane)
    const int a_row = tid / (GM_BK / GM_EA), a_k = (tid % (GM_BK / GM_EA)) * GM_EA;
    const int b_k = tid / (GM_BN / GM_EB), b_col = (tid % (GM_BN / GM_EB)) * GM_EB;
    double ra[GM_EA], rb[GM_EB];

    auto load_tiles = [&](int64_t k0) {
        const int64_t gm = m0 + a_row;
        const double *ap = A + gm * K + k0 + a_k;
#pragma unroll
        for (int e = 0; e < GM_EA; ++e) {
            if (GUARD)
                ra[e] = (gm < M && k0 + a_k + e < K) ? ap[e] : 0.0;
            else
                ra[e] = ap[e];
        }
        const int64_t gk = k0 + b_k;
        const double *bp = B + gk * N + n0 + b_col;
#pragma unroll
        for (int e = 0; e < GM_EB; ++e) {
            if (GUARD)
                rb[e] = (gk < K && n0 + b_col + e < N) ? bp[e] : 0.0;
            else
                rb[e] = bp[e];
        }
    };
    auto store_tiles = [&](int buf) {
#pragma unroll
        for (int e = 0; e < GM_EA; ++e)
            As[buf][a_k + e][a_row] = ra[e];
#pragma unroll
        for (int e = 0; e < GM_EB; ++e)
            Bs[buf][b_k][b_col + e] = rb[e];
    };

    double4_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            acc[i][j] = (double4_t){0.0, 0.0, 0.0, 0.0};

    const int64_t nk = (K + GM_BK - 1) / GM_BK;
    load_tiles(0);
    store_tiles(0);
    __syncthreads();
    const int fr = lane & 15, fk = lane >> 4;
    for (int64_t kt = 0; kt < nk; ++kt) {
        const int cur = (int)(kt & 1);
        if (kt + 1 < nk)
            load_tiles((kt + 1) * GM_BK);
#pragma unroll
        for (int ks = 0; ks < GM_BK; ks += 4) {
            double af[4], bf[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                af[i] = As[cur][ks + fk][wm * 64 + i * 16 + fr];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                bf[j] = Bs[cur][ks + fk][wn * 64 + j * 16 + fr];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk)
            store_tiles(cur ^ 1);
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int64_t gm = m0 + wm * 64 + i * 16 + 4 * v + fk;
                const int64_t gn = n0 + wn * 64 + j * 16 + fr;
                if (!GUARD || (gm < M && gn < N)) {
                    double r = acc[i][j][v];
                    if (use_c)
                        r = C[gm * N + gn] + r;
                    C[gm * N + gn] = r;
                }
            }
}

static int dgemm_device(int64_t M, int64_t N, int64_t K, const double *A, const double *B, double *C, double beta)
{
    if (M < 0 || N < 0 || K < 0)
        return set_error(COMET_HIP_ERR_ARG, "negative GEMM size");
    if (beta != 0.0 && beta != 1.0)
        return set_error(COMET_HIP_ERR_ARG, "beta must be 0 or 1 (got %g)", beta);
    if (M == 0 || N == 0)
        return COMET_HIP_OK;
    const int64_t gx = ceil_div(N, GM_BN), gy = ceil_div(M, GM_BM);
    if (gy > 65535)
        return set_error(COMET_HIP_ERR_SIZE, "M = %lld too large for the launch grid", (long long)M);
    const bool aligned = (M % GM_BM == 0) && (N % GM_BN == 0) && (K % GM_BK == 0) && K > 0;
    KernelTimer t("dgemm_mfma_kernel");
    if (aligned)
        dgemm_mfma_kernel<false><<<dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, stream()>>>(M, N, K, A, B, C,
                                                                                             beta != 0.0);
    else
        dgemm_mfma_kernel<true><<<dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, stream()>>>(M, N, K, A, B, C,
                                                                                            beta != 0.0);
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}

// ============================================================================
// Plan
// ============================================================================
static bool contains(const int32_t *v, int n, int32_t x)
{
    for (int i = 0; i < n; ++i)
        if (v[i] == x)
            return true;
    return false;
}

// position in `in` of each element of `out` (Utils.h:722-733)
static void positions_of(const int32_t *in, const int32_t *out, int n, int32_t *perm)
{
    for (int i = 0; i < n; ++i)
        perm[i] = (int32_t)(std::find(in, in + n, out[i]) - in);
}

static int make_plan(int32_t rankA, const int32_t *a_lab, int32_t rankB, const int32_t *b_lab, int32_t rankC,
                     const int32_t *c_lab, const int64_t *extent, int32_t which, comet_ttgt_plan *plan)
{
    if (rankA < 1 || rankB < 1 || rankC < 1 || rankA > 8 || rankB > 8 || rankC > 8)
        return set_error(COMET_HIP_ERR_ARG, "tensor rank outside [1,8]");
    std::vector<int32_t> m, n, k;
    for (int i = 0; i < rankA; ++i) {
        if (contains(c_lab, rankC, a_lab[i])) {
            if (contains(b_lab, rankB, a_lab[i]))
                return set_error(COMET_HIP_ERR_ARG, "label %d appears in A, B and C: not a TTGT contraction", a_lab[i]);
            m.push_back(a_lab[i]);
        } else {
            k.push_back(a_lab[i]);
        }
    }
    for (int i = 0; i < rankB; ++i) {
        if (contains(c_lab, rankC, b_lab[i]))
            n.push_back(b_lab[i]);
        else if (!contains(a_lab, rankA, b_lab[i]))
            return set_error(COMET_HIP_ERR_ARG, "label %d of B is neither contracted with A nor kept in C", b_lab[i]);
    }
    for (int32_t x : k)
        if (!contains(b_lab, rankB, x))
            return set_error(COMET_HIP_ERR_ARG, "label %d of A is neither contracted with B nor kept in C", x);
    if ((int)(m.size() + k.size()) != rankA || (int)(n.size() + k.size()) != rankB ||
        (int)(m.size() + n.size()) != rankC)
        return set_error(COMET_HIP_ERR_ARG, "index sets do not form a GEMM (repeated or missing labels)");
    std::sort(m.begin(), m.end());
    std::sort(n.begin(), n.end());
    std::sort(k.begin(), k.end());
    int64_t M = 1, N = 1, K = 1;
    for (int32_t x : m) M *= extent[x];
    for (int32_t x : n) N *= extent[x];
    for (int32_t x : k) K *= extent[x];
    const double a_size = (double)(K * M), b_size = (double)(N * K), c_size = (double)(M * N);
    auto cost_of = [](double size, const int32_t *perm) { return perm[0] != 0 ? size / 0.71 : size; };

    int32_t cand = 0;
    bool have = false;
    double best = 0.0;
    do {
        do {
            do {
                for (int sw = 0; sw < 2; ++sw) {
                    comet_ttgt_plan cur;
                    std::memset(&cur, 0, sizeof cur);
                    cur.rankA = rankA;
                    cur.rankB = rankB;
                    cur.rankC = rankC;
                    std::vector<int32_t> ai, bi, ci;
                    if (sw) {
                        ai = k; ai.insert(ai.end(), m.begin(), m.end());
                        bi = n; bi.insert(bi.end(), k.begin(), k.end());
                        ci = n; ci.insert(ci.end(), m.begin(), m.end());
                    } else {
                        ai = m; ai.insert(ai.end(), k.begin(), k.end());
                        bi = k; bi.insert(bi.end(), n.begin(), n.end());
                        ci = m; ci.insert(ci.end(), n.begin(), n.end());
                    }
                    std::copy(ai.begin(), ai.end(), cur.a_idx);
                    std::copy(bi.begin(), bi.end(), cur.b_idx);
                    std::copy(ci.begin(), ci.end(), cur.c_idx);
                    positions_of(a_lab, cur.a_idx, rankA, cur.permA);
                    positions_of(b_lab, cur.b_idx, rankB, cur.permB);
                    positions_of(c_lab, cur.c_idx, rankC, cur.permC);
                    cur.transA = !std::equal(ai.begin(), ai.end(), a_lab);
                    cur.transB = !std::equal(bi.begin(), bi.end(), b_lab);
                    cur.transC = !std::equal(ci.begin(), ci.end(), c_lab);
                    cur.swapAB = sw;
                    cur.M = M;
                    cur.N = N;
                    cur.K = K;
                    double t = 0.0;
                    if (cur.transA) t = t + cost_of(a_size, cur.permA);
                    if (cur.transB) t = t + cost_of(b_size, cur.permB);
                    if (cur.transC) t = t + cost_of(c_size, cur.permC);
                    cur.cost = t;
                    cur.candidate = cand;
                    const bool take = which >= 0 ? cand == which : (!have || t < best);
                    if (take) {
                        *plan = cur;
                        best = t;
                        have = true;
                    }
                    ++cand;
                }
            } while (std::next_permutation(k.begin(), k.end()));
        } while (std::next_permutation(n.begin(), n.end()));
    } while (std::next_permutation(m.begin(), m.end()));
    if (which >= cand || !have)
        return set_error(COMET_HIP_ERR_ARG, "candidate %d does not exist (%d candidates)", which, cand);
    plan->ncandidates = cand;
    return COMET_HIP_OK;
}

static Workspace g_tt_a, g_tt_b, g_tt_c;

}  // namespace comet

using namespace comet;

extern "C" int comet_hip_transpose_f64(int32_t rank, const int64_t *in_shape, const int32_t *perm, int64_t in_dptr,
                                       int64_t out_dptr)
{
    COMET_CHK(ensure_init());
    if (!in_shape || !perm || !in_dptr || !out_dptr)
        return set_error(COMET_HIP_ERR_ARG, "null argument to comet_hip_transpose_f64");
    if (in_dptr == out_dptr)
        return set_error(COMET_HIP_ERR_ARG, "in-place transpose is not supported");
    return transpose_device(rank, in_shape, perm, (const double *)in_dptr, (double *)out_dptr);
}

extern "C" int comet_hip_dgemm_f64(int64_t M, int64_t N, int64_t K, int64_t a_dptr, int64_t b_dptr, int64_t c_dptr,
                                   double beta)
{
    COMET_CHK(ensure_init());
    if ((M > 0 && N > 0 && !c_dptr) || (M > 0 && N > 0 && K > 0 && (!a_dptr || !b_dptr)))
        return set_error(COMET_HIP_ERR_ARG, "null matrix passed to comet_hip_dgemm_f64");
    return dgemm_device(M, N, K, (const double *)a_dptr, (const double *)b_dptr, (double *)c_dptr, beta);
}

extern "C" int comet_hip_ttgt_plan(int32_t rankA, const int32_t *a_lab, int32_t rankB, const int32_t *b_lab,
                                   int32_t rankC, const int32_t *c_lab, const int64_t *extent, int32_t which,
                                   comet_ttgt_plan *plan)
{
    if (!a_lab || !b_lab || !c_lab || !extent || !plan)
        return set_error(COMET_HIP_ERR_ARG, "null argument to comet_hip_ttgt_plan");
    return make_plan(rankA, a_lab, rankB, b_lab, rankC, c_lab, extent, which, plan);
}

// Yardstick for the GEMM: back-to-back v_mfma_f64_16x16x4_f64 on registers only, sixteen independent
// accumulators per wavefront (more than the instruction's latency needs), two wavefronts per SIMD on every CU.
__global__ __launch_bounds__(256, 2) void mfma_f64_peak_kernel(int64_t iters, double *__restrict__ out)
{
    double4_t acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
        acc[i] = (double4_t){0.0, 0.0, 0.0, 0.0};
    const double a = 1.0 + threadIdx.x * 1e-9, b = 1.0 - threadIdx.x * 1e-9;
    for (int64_t it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 16; ++i)
            acc[i] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, acc[i], 0, 0, 0);
    }
    double4_t s = acc[0];
#pragma unroll
    for (int i = 1; i < 16; ++i)
        s += acc[i];
    out[(int64_t)blockIdx.x * blockDim.x + threadIdx.x] = s[0] + s[1] + s[2] + s[3];
}

static Workspace g_peak_out;

extern "C" int comet_hip_mfma_f64_peak(int64_t iters, double *tflops)
{
    COMET_CHK(ensure_init());
    if (iters <= 0 || iters > (1ll << 24) || !tflops)
        return set_error(COMET_HIP_ERR_ARG, "bad arguments to comet_hip_mfma_f64_peak");
    const int blocks = num_cus() * 2;        // 8 wavefronts per CU: two per SIMD
    COMET_CHK(g_peak_out.ensure(sizeof(double) * 256 * (size_t)blocks, false));
    hipEvent_t e0, e1;
    COMET_HIPCHK(hipEventCreate(&e0));
    COMET_HIPCHK(hipEventCreate(&e1));
    float best = 0.f;
    for (int rep = 0; rep < 4; ++rep) {      // the first launch warms the clocks up
        COMET_HIPCHK(hipEventRecord(e0, stream()));
        mfma_f64_peak_kernel<<<dim3((unsigned)blocks), dim3(256), 0, stream()>>>(iters, (double *)g_peak_out.ptr);
        COMET_HIPCHK(hipEventRecord(e1, stream()));
        COMET_HIPCHK(hipEventSynchronize(e1));
        float ms = 0.f;
        COMET_HIPCHK(hipEventElapsedTime(&ms, e0, e1));
        if (rep > 0 && (best == 0.f || ms < best))
            best = ms;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    COMET_HIPCHK(hipGetLastError());
    const double flops = 2.0 * 16 * 16 * 4 * 16.0 * (double)iters * 4.0 * blocks;      // per MFMA x 16 x iters x waves
    *tflops = flops / ((double)best * 1e-3) / 1e12;
    return COMET_HIP_OK;
}

extern "C" int comet_hip_ttgt_contract(const comet_ttgt_plan *plan, const int64_t *a_shape, const int64_t *b_shape,
                                       const int64_t *c_shape, int64_t a_dptr, int64_t b_dptr, int64_t c_dptr,
                                       double beta)
{
    COMET_CHK(ensure_init());
    if (!plan || !a_shape || !b_shape || !c_shape || !a_dptr || !b_dptr || !c_dptr)
        return set_error(COMET_HIP_ERR_ARG, "null argument to comet_hip_ttgt_contract");
    if (beta != 0.0 && beta != 1.0)
        return set_error(COMET_HIP_ERR_ARG, "beta must be 0 or 1 (got %g)", beta);
    // the plan may come from anywhere: ranks index 8-entry arrays and each perm must be a permutation
    auto is_perm = [](const int32_t *perm, int rank) {
        unsigned seen = 0;
        for (int i = 0; i < rank; ++i) {
            if (perm[i] < 0 || perm[i] >= rank || (seen >> perm[i] & 1u))
                return false;
            seen |= 1u << perm[i];
        }
        return true;
    };
    if (plan->rankA < 1 || plan->rankA > 8 || plan->rankB < 1 || plan->rankB > 8 || plan->rankC < 1 || plan->rankC > 8)
        return set_error(COMET_HIP_ERR_ARG, "plan ranks (%d, %d, %d) outside 1..8", plan->rankA, plan->rankB,
                         plan->rankC);
    if ((plan->transA && !is_perm(plan->permA, plan->rankA)) || (plan->transB && !is_perm(plan->permB, plan->rankB)) ||
        (plan->transC && !is_perm(plan->permC, plan->rankC)))
        return set_error(COMET_HIP_ERR_ARG, "a transpose of the plan is not a permutation of its tensor's dimensions");
    const int64_t M = plan->M, N = plan->N, K = plan->K;
    if (M < 0 || N < 0 || K < 0)
        return set_error(COMET_HIP_ERR_ARG, "negative GEMM extent in the plan");
    int64_t ta = 1, tb = 1, tc = 1;
    for (int i = 0; i < plan->rankA; ++i) ta *= a_shape[i];
    for (int i = 0; i < plan->rankB; ++i) tb *= b_shape[i];
    for (int i = 0; i < plan->rankC; ++i) tc *= c_shape[i];
    if (ta != M * K || tb != K * N || tc != M * N)
        return set_error(COMET_HIP_ERR_ARG, "tensor shapes do not match the plan (M,N,K = %lld,%lld,%lld)",
                         (long long)M, (long long)N, (long long)K);
    const double *A = (const double *)a_dptr, *B = (const double *)b_dptr;
    double *C = (double *)c_dptr;
    const double *Ause = A, *Buse = B;
    double *Cuse = C;
    if (plan->transA) {
        COMET_CHK(g_tt_a.ensure(sizeof(double) * (size_t)ta, false));
        COMET_CHK(transpose_device(plan->rankA, a_shape, plan->permA, A, (double *)g_tt_a.ptr));
        Ause = (const double *)g_tt_a.ptr;
    }
    if (plan->transB) {
        COMET_CHK(g_tt_b.ensure(sizeof(double) * (size_t)tb, false));
        COMET_CHK(transpose_device(plan->rankB, b_shape, plan->permB, B, (double *)g_tt_b.ptr));
        Buse = (const double *)g_tt_b.ptr;
    }
    double gemm_beta = beta;
    if (plan->transC) {
        COMET_CHK(g_tt_c.ensure(sizeof(double) * (size_t)tc, false));
        Cuse = (double *)g_tt_c.ptr;
        if (beta != 0.0)
            COMET_CHK(transpose_device(plan->rankC, c_shape, plan->permC, C, Cuse));
    }
    if (plan->swapAB)
        COMET_CHK(dgemm_device(N, M, K, Buse, Ause, Cuse, gemm_beta));
    else
        COMET_CHK(dgemm_device(M, N, K, Ause, Buse, Cuse, gemm_beta));
    if (plan->transC) {
        int64_t cp_shape[8];
        int32_t rev[8];
        for (int i = 0; i < plan->rankC; ++i) {
            cp_shape[i] = c_shape[plan->permC[i]];
            rev[plan->permC[i]] = i;
        }
        COMET_CHK(transpose_device(plan->rankC, cp_shape, rev, Cuse, C));
    }
    return COMET_HIP_OK;
}
