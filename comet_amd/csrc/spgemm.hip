// Gustavson SpGEMM (symbolic + numeric), masked SpGEMM and the fused
// masked-SpGEMM + SUM used for triangle counting, for gfx950.
//
// What is computed is what the reference's workspace lowering computes
// (lib/Dialect/IndexTree/Transforms/SymbolicCompute.cpp:215-339,
// lib/Conversion/IndexTreeToSCF/SymbolicDomainConversion.cpp:81-340,
// lib/Dialect/IndexTree/Transforms/WorkspaceTransforms.cpp:97-276,
// lib/Conversion/TensorAlgebraToSCF/SparseTensorConversionPass.cpp:595-638,
// 982-1159; masks: lib/Conversion/IndexTreeToSCF/IndexTreeToSCF.cpp:1083-1148,
// 1327-1448): every structurally reachable (i,j) is kept, columns come out
// ascending.  How it is computed is different: one 1024-lane workgroup owns a
// row at a time and keeps the row's column set as a bitmap in LDS (128 KiB
// covers 2^20 columns), so counting is a popcount, "sort the touched columns"
// (the reference's comet_sort call) is reading the bitmap in order, and the
// mark array / mark value bookkeeping disappears.  Values accumulate with
// fp64 atomics, in one of three places chosen by the number of products of the
// row: a dense per-workgroup slab in HBM (few products, every masked product and
// every semiring other than plus-times; the extraction step reads it back and
// re-zeroes it with an atomic exchange, so every access to the slab is performed
// at the L2 and no stale L1 line can be seen), a compact array in LDS indexed by
// the rank of the column among the row's columns (spgemm_numeric_span_kernel),
// or LDS accumulators for one block of 16384 columns at a time
// (spgemm_numeric_dense_kernel, the widest rows).
// The order in which the products of one (i,j) are added is therefore not the
// reference's ascending-k order: values agree to rounding, structure exactly.
#include <type_traits>

#include "common.h"
#include <cstring>

namespace comet {

// Coalesced stores of C go out as streaming (non-temporal) stores: C is written once and never read here, and
// its 289 GB at scale 20 would otherwise push the rows of B out of the L2 (-7 ms in the block kernel, -7 ms in
// the span kernel).  Stores that scatter, a few bytes per lane - the span kernel's columns - stay ordinary:
// as streaming stores they reach memory unmerged (span kernel 144 -> 411 ms).
template <typename T>
__device__ __forceinline__ void store_streaming(T *p, T v)
{
    __builtin_nontemporal_store(v, p);
}

constexpr int SG_T = 1024;                 // lanes per workgroup
constexpr int SG_WAVES = SG_T / 64;
constexpr int SG_LDS_MAX_W = 32;           // words per lane that still fit LDS (33 * 1024 * 4 B = 132 KiB)

__device__ inline int64_t readlane_i64(int64_t v, int lane)
{
    int lo = (int)(v & 0xffffffff), hi = (int)(v >> 32);
    lo = __builtin_amdgcn_readlane(lo, lane);
    hi = __builtin_amdgcn_readlane(hi, lane);
    return ((int64_t)hi << 32) | (uint32_t)lo;
}

__device__ inline double readlane_d(double v, int lane)
{
    int lo = __double2loint(v), hi = __double2hiint(v);
    lo = __builtin_amdgcn_readlane(lo, lane);
    hi = __builtin_amdgcn_readlane(hi, lane);
    return __hiloint2double(hi, lo);
}

// Bitmap layout: word w = j/32 sits at address w + w/W, i.e. one padding word
// after every W words, W = words per lane.  Random probes of neighbouring
// columns land in neighbouring LDS banks, and the extraction sweep, in which
// lane t reads its own words t*W .. t*W+W-1 at addresses t*(W+1)+k, is
// conflict-free too because W+1 is odd.
struct BmAddr {
    int logW;
    __device__ inline int word(int j) const
    {
        const int w = j >> 5;
        return w + (w >> logW);
    }
    __device__ inline uint32_t bit(int j) const { return 1u << (j & 31); }
};

// Visit every product of output row i: f(j, q, a, p, s) for k = Acrd[p] in A_i,
// q over the entries [s, e) of B_k, j = Bcrd[q], a = A's value (the visitor
// loads Bval[q] itself, and only if it needs it).  The entries of A_i are dealt to the 16 wavefronts
// one at a time (entry p goes to wavefront p mod 16), because in a sorted row
// the neighbours with long rows sit next to each other and would otherwise all
// land on one wavefront.  A wavefront fetches 64 of its entries at once (one per
// lane).  Rows of B with at least FEP_SHORT entries are then walked one by one
// with all lanes striding over B_k; shorter ones go to the four 16-lane quarters,
// four rows at a time.  A wavefront runs these turns one after the other and a
// turn costs about one trip to memory, so each turn issues all of its loads (up
// to four per lane; a load no lane needs is skipped) before the visitor runs.
constexpr int FEP_SHORT = 32, FEP_SHORT_LOADS = FEP_SHORT / 16, FEP_LONG_LOADS = 4;
constexpr int FEP_WIDE_DEPTH = 4;       // turns of a long row a wavefront takes at a time (WIDE walks)
// what the look-up and fetch steps of a masked product's visitor hand to the visit itself: where the column's
// value lives (negative: the mask does not hold the column) and B's value, fetched for hits only
struct MaskHit {
    int at;
    double b;
};
// four consecutive entries of an index array that lies at any 4-byte boundary
typedef int sg_i4u __attribute__((ext_vector_type(4), aligned(4)));
// With WIDE, a lane takes four consecutive entries in a turn in which every lane has all its entries - one 16-byte
// load instead of four loads 64 entries apart - and f4(j, q, a, p, s) visits the entries q .. q + 3 of B_k at once
// (their columns in j).  That pays where the visitor can treat neighbouring columns together (the symbolic phase:
// 78 -> 64 ms on A*A of an R-MAT graph of scale 20); a visitor that probes a hash table per product is slower with
// it (masked numeric phase, 247 -> 300 ms).
// A visitor that looks its column up in LDS first (a mask's bitmap or hash table) and fetches B's value only on a
// hit hands these two steps in as pre(j) and mid(j, q, what pre returned), and f gets what mid returned as a sixth
// argument.  The walk runs pre for all the entries of a turn together, then mid for all of them (inside f each
// step would sit behind the branch of the entry before it: four trips to LDS and four to memory per turn, one
// after the other) - and it visits a turn's entries one turn late, after the next turn's columns have arrived and
// its look-ups are out, so that the trip to memory for the values of the hits overlaps with the next turn's instead
// of standing alone (a wavefront runs its turns one after the other, and nothing else hides that trip).  The
// look-ups of a turn therefore run before the visits of the turn before it: they must not depend on them.
template <bool VALUES, bool WIDE, typename PRE, typename MID, typename F, typename F4>
__device__ inline void for_each_product_impl(int64_t as, int64_t ae, const int32_t *__restrict__ Acrd,
                                             const double *__restrict__ Aval, const int64_t *__restrict__ Bpos,
                                             const int32_t *__restrict__ Bcrd, PRE pre, MID mid, F f, F4 f4)
{
    using T1 = decltype(pre(0));
    using T2 = decltype(mid(0, (int64_t)0, T1()));
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int quarter = lane >> 4, sub = lane & 15;
    // the entries of the turn before: visited once the next turn's look-ups are out
    constexpr int NP = FEP_LONG_LOADS > FEP_SHORT_LOADS ? FEP_LONG_LOADS : FEP_SHORT_LOADS;
    bool w_ok[NP];
    int w_j[NP];
    int64_t w_q[NP], w_p[NP], w_s[NP];
    double w_a[NP];
    T2 w_md[NP];
#pragma unroll
    for (int x = 0; x < NP; ++x)
        w_ok[x] = false;
    const auto visit_pending = [&]() {
#pragma unroll
        for (int x = 0; x < NP; ++x)
            if (w_ok[x])
                f(w_j[x], w_q[x], w_a[x], w_p[x], w_s[x], w_md[x]);
    };
    // one turn: up to N entries per lane (ok[x]: the lane has entry x), columns j, places q in B
    const auto turn = [&](auto n_tag, const bool *ok, const int *j, const int64_t *q, double at, int64_t p, int64_t s) {
        constexpr int N = decltype(n_tag)::value;
        T1 tk[N];
#pragma unroll
        for (int x = 0; x < N; ++x)
            tk[x] = ok[x] ? pre(j[x]) : T1();
        visit_pending();
#pragma unroll
        for (int x = 0; x < NP; ++x) {
            w_ok[x] = x < N ? ok[x] : false;
            if (x < N) {
                w_j[x] = j[x];
                w_q[x] = q[x];
                w_a[x] = at;
                w_p[x] = p;
                w_s[x] = s;
                w_md[x] = ok[x] ? mid(j[x], q[x], tk[x]) : T2();
            }
        }
    };
    for (int64_t base = as + wave; base < ae; base += (int64_t)SG_WAVES * 64) {
        const int64_t left = (ae - base + SG_WAVES - 1) / SG_WAVES;     // my entries from here on
        const int cnt = (int)(left < 64 ? left : 64);
        int64_t bs = 0, be = 0;
        double a = 0.0;
        if (lane < cnt) {
            const int64_t p = base + (int64_t)lane * SG_WAVES;
            const int k = Acrd[p];
            bs = Bpos[k];
            be = Bpos[k + 1];
            if (VALUES)
                a = Aval[p];
        }
        unsigned long long big = __ballot(be - bs >= FEP_SHORT);
        unsigned long long todo = __ballot(bs < be && be - bs < FEP_SHORT);
        while (big) {
            const int t = __builtin_ctzll(big);
            big &= big - 1;
            const int64_t s = readlane_i64(bs, t), len = readlane_i64(be, t) - s;
            const double at = VALUES ? readlane_d(a, t) : 0.0;
            const int64_t p = base + (int64_t)t * SG_WAVES;
            int64_t o = lane;
            if (WIDE && len >= 64 * FEP_LONG_LOADS) {
                // Turns in which every lane has all its entries: a lane takes four consecutive ones, a single
                // 16-byte load, and the loads of the next turn are in flight while the visitor works on this one.
                static_assert(FEP_LONG_LOADS == 4, "a lane's entries of a full turn are one 16-byte load");
                int64_t c = s + 4 * (int64_t)lane;
                int64_t done = 0;
                // A wavefront with one or two kilobytes on their way from memory waits most of the time (a row of
                // B comes from beyond the L2 as a rule, two microseconds away): rows long enough are taken
                // FEP_WIDE_DEPTH turns at a time with as many again in flight behind them, then two at a time
                // (symbolic phase of A*A on an R-MAT graph of scale 20: 64.7 -> 46.8 ms; eight at a time gains
                // nothing over four).
                constexpr int64_t TURN = 64 * FEP_LONG_LOADS;
                const auto deep = [&](auto dtag) {
                    constexpr int D = decltype(dtag)::value;
                    if (len - done < 2 * D * TURN)
                        return;
                    sg_i4u jd[D];
#pragma unroll
                    for (int d = 0; d < D; ++d)
                        jd[d] = *reinterpret_cast<const sg_i4u *>(Bcrd + c + d * TURN);
                    for (int64_t full = done + D * TURN; full + D * TURN <= len; full += D * TURN) {
                        sg_i4u jn[D];
#pragma unroll
                        for (int d = 0; d < D; ++d)
                            jn[d] = *reinterpret_cast<const sg_i4u *>(Bcrd + c + (D + d) * TURN);
#pragma unroll
                        for (int d = 0; d < D; ++d)
                            f4(jd[d], c + d * TURN, at, p, s);
#pragma unroll
                        for (int d = 0; d < D; ++d)
                            jd[d] = jn[d];
                        c += D * TURN;
                        done += D * TURN;
                    }
#pragma unroll
                    for (int d = 0; d < D; ++d)
                        f4(jd[d], c + d * TURN, at, p, s);
                    c += D * TURN;
                    done += D * TURN;
                };
                deep(std::integral_constant<int, FEP_WIDE_DEPTH>());
                deep(std::integral_constant<int, 2>());
                if (len - done >= TURN) {
                sg_i4u j = *reinterpret_cast<const sg_i4u *>(Bcrd + c);
                for (int64_t full = done + 64 * FEP_LONG_LOADS; full + 64 * FEP_LONG_LOADS <= len;
                     full += 64 * FEP_LONG_LOADS) {
                    const sg_i4u jn = *reinterpret_cast<const sg_i4u *>(Bcrd + c + 64 * FEP_LONG_LOADS);
                    f4(j, c, at, p, s);
                    j = jn;
                    c += 64 * FEP_LONG_LOADS;
                    done += 64 * FEP_LONG_LOADS;
                }
                f4(j, c, at, p, s);
                done += 64 * FEP_LONG_LOADS;
                }
                o += done;
            }
            if (!WIDE && len >= 64 * FEP_LONG_LOADS) {
                // Turns in which every lane has all its entries: no predicates, and the loads of the next such
                // turn are in flight while this one's look-ups and the visits of the turn before it run.
                bool all[FEP_LONG_LOADS];
                int j[FEP_LONG_LOADS];
                int64_t q[FEP_LONG_LOADS];
#pragma unroll
                for (int x = 0; x < FEP_LONG_LOADS; ++x) {
                    all[x] = true;
                    j[x] = Bcrd[s + o + 64 * x];
                }
                for (int64_t full = 64 * FEP_LONG_LOADS; full + 64 * FEP_LONG_LOADS <= len;
                     full += 64 * FEP_LONG_LOADS) {
                    int jn[FEP_LONG_LOADS];
#pragma unroll
                    for (int x = 0; x < FEP_LONG_LOADS; ++x)
                        jn[x] = Bcrd[s + o + 64 * (FEP_LONG_LOADS + x)];
#pragma unroll
                    for (int x = 0; x < FEP_LONG_LOADS; ++x)
                        q[x] = s + o + 64 * x;
                    turn(std::integral_constant<int, FEP_LONG_LOADS>(), all, j, q, at, p, s);
#pragma unroll
                    for (int x = 0; x < FEP_LONG_LOADS; ++x)
                        j[x] = jn[x];
                    o += 64 * FEP_LONG_LOADS;
                }
#pragma unroll
                for (int x = 0; x < FEP_LONG_LOADS; ++x)
                    q[x] = s + o + 64 * x;
                turn(std::integral_constant<int, FEP_LONG_LOADS>(), all, j, q, at, p, s);
                o += 64 * FEP_LONG_LOADS;
            }
            if (o < len) {          // the rest of the row: fewer than 64 * FEP_LONG_LOADS entries
                bool ok[FEP_LONG_LOADS];
                int j[FEP_LONG_LOADS];
                int64_t q[FEP_LONG_LOADS];
#pragma unroll
                for (int x = 0; x < FEP_LONG_LOADS; ++x) {
                    ok[x] = o + 64 * x < len;
                    q[x] = s + o + 64 * x;
                }
#pragma unroll
                for (int x = 0; x < FEP_LONG_LOADS; ++x)
                    j[x] = ok[x] ? Bcrd[q[x]] : 0;
                turn(std::integral_constant<int, FEP_LONG_LOADS>(), ok, j, q, at, p, s);
            }
        }
        while (todo) {
            int pick = -1;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int t = todo ? __builtin_ctzll(todo) : -1;
                todo = todo ? (todo & (todo - 1)) : 0;
                pick = quarter == g ? t : pick;
            }
            const int src = pick < 0 ? lane : pick;
            const int64_t s = ((int64_t)__shfl((int)(bs >> 32), src, 64) << 32) |
                              (uint32_t)__shfl((int)(bs & 0xffffffff), src, 64);
            const int64_t e = ((int64_t)__shfl((int)(be >> 32), src, 64) << 32) |
                              (uint32_t)__shfl((int)(be & 0xffffffff), src, 64);
            const double at =
                VALUES ? __hiloint2double(__shfl(__double2hiint(a), src, 64), __shfl(__double2loint(a), src, 64)) : 0.0;
            const int64_t p = base + (int64_t)src * SG_WAVES;
            bool ok[FEP_SHORT_LOADS];
            int j[FEP_SHORT_LOADS];
            int64_t q[FEP_SHORT_LOADS];
#pragma unroll
            for (int x = 0; x < FEP_SHORT_LOADS; ++x) {
                ok[x] = pick >= 0 && s + sub + 16 * x < e;
                q[x] = s + sub + 16 * x;
            }
#pragma unroll
            for (int x = 0; x < FEP_SHORT_LOADS; ++x)
                j[x] = ok[x] ? Bcrd[q[x]] : 0;
            turn(std::integral_constant<int, FEP_SHORT_LOADS>(), ok, j, q, at, p, s);
        }
    }
    visit_pending();
}

template <bool VALUES, typename F>
__device__ inline void for_each_product(int64_t as, int64_t ae, const int32_t *__restrict__ Acrd,
                                        const double *__restrict__ Aval, const int64_t *__restrict__ Bpos,
                                        const int32_t *__restrict__ Bcrd, F f)
{
    for_each_product_impl<VALUES, false>(
        as, ae, Acrd, Aval, Bpos, Bcrd, [](int) { return 0u; }, [](int, int64_t, uint32_t) { return 0u; },
        [&](int j, int64_t q, double a, int64_t p, int64_t s, uint32_t) { f(j, q, a, p, s); },
        [](sg_i4u, int64_t, double, int64_t, int64_t) {});
}
template <bool VALUES, typename PRE, typename MID, typename F>
__device__ inline void for_each_product_probed(int64_t as, int64_t ae, const int32_t *__restrict__ Acrd,
                                               const double *__restrict__ Aval, const int64_t *__restrict__ Bpos,
                                               const int32_t *__restrict__ Bcrd, PRE pre, MID mid, F f)
{
    for_each_product_impl<VALUES, false>(as, ae, Acrd, Aval, Bpos, Bcrd, pre, mid, f,
                                         [](sg_i4u, int64_t, double, int64_t, int64_t) {});
}
template <bool VALUES, typename F, typename F4>
__device__ inline void for_each_product(int64_t as, int64_t ae, const int32_t *__restrict__ Acrd,
                                        const double *__restrict__ Aval, const int64_t *__restrict__ Bpos,
                                        const int32_t *__restrict__ Bcrd, F f, F4 f4)
{
    for_each_product_impl<VALUES, true>(
        as, ae, Acrd, Aval, Bpos, Bcrd, [](int) { return 0u; }, [](int, int64_t, uint32_t) { return 0u; },
        [&](int j, int64_t q, double a, int64_t p, int64_t s, uint32_t) { f(j, q, a, p, s); }, f4);
}

__device__ inline int wave_sum_i32(int v)
{
    for (int d = 32; d > 0; d >>= 1)
        v += __shfl_down(v, d, 64);
    return v;
}

__device__ inline double wave_sum_f64(double v)
{
    for (int d = 32; d > 0; d >>= 1)
        v += __shfl_down(v, d, 64);
    return v;
}

// Rows are handed out through a global ticket counter, because row costs differ
// by six orders of magnitude and follow the bit pattern of the row id in R-MAT
// graphs (a fixed row -> workgroup map leaves some workgroups with ten times the
// work of others).  Lane 0 draws the ticket, LDS broadcasts it, and the value is
// read back through readfirstlane so that it lives in scalar registers: every
// branch on the row index is then a uniform scalar branch.  That matters because
// the row loop contains workgroup barriers.  The loop must also keep a single
// back edge with the draw at its end (no `continue`): with a draw at the top and
// a `continue` below it the compiler splits the loop per lane and parks lanes
// 1..1023 in a barrier loop that never draws again, which hangs the workgroup.
// What a ticket indexes is a list of the rows that have work, heaviest first
// (RowList): empty rows and rows another kernel serves cost no ticket, and the
// rows that take milliseconds start first instead of forming the tail.
struct RowList {
    const int32_t *rows;       // row - row_begin, by descending number of products
    const int64_t *bounds;     // [0] rows with >= dense_threshold products, [1] rows with any product,
                               // [2] rows with >= wide_threshold products (a prefix of [0])
};
__device__ inline void list_range(const RowList &l, int part, int64_t *first, int64_t *end)
{
    // part 0: the heavy rows, 1: the others that have products, 2: both, 3: the widest of the heavy rows,
    // 4: the heavy rows that are not among the widest
    *first = part == 1 ? l.bounds[0] : part == 4 ? l.bounds[2] : 0;
    *end = part == 0 || part == 4 ? l.bounds[0] : part == 3 ? l.bounds[2] : l.bounds[1];
}
// A workgroup barrier that orders LDS traffic only.  __syncthreads() also makes every wavefront wait until its
// global stores have been acknowledged, a microsecond that a kernel whose stores nobody reads back (the rows
// of C going out) need not spend at every barrier.
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}
// Inclusive prefix sum over the 64 lanes of a wavefront through the cross-lane data path of the vector ALU
// (shifts within a row of 16 lanes, then the last lane of a row broadcast to the rows after it): no LDS round
// trips, unlike a shuffle.  A lane whose source lies outside its row, or whose row is masked, adds 0.
__device__ __forceinline__ int wave_inclusive_scan(int v)
{
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);    // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);    // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);    // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);    // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);    // row_bcast:15 into rows 1 and 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);    // row_bcast:31 into rows 2 and 3
    return v;
}
template <bool LDS_ONLY = false>
__device__ inline int64_t draw_row(unsigned long long *ticket, int64_t first, int64_t *slot)
{
    if (threadIdx.x == 0)
        *slot = first + (int64_t)atomicAdd(ticket, 1ull);
    if (LDS_ONLY)
        lds_barrier();
    else
        __syncthreads();
    const int64_t r = *slot;
    if (LDS_ONLY)
        lds_barrier();
    else
        __syncthreads();
    const int lo = __builtin_amdgcn_readfirstlane((int)(r & 0xffffffff));
    const int hi = __builtin_amdgcn_readfirstlane((int)(r >> 32));
    return ((int64_t)hi << 32) | (uint32_t)lo;
}

// Two kernels that share one list, one taking rows from its front and one from its back until they meet: the
// ticket word holds both counts (front in the low half, back in the high half), so the value an atomic add
// returns tells the claimant how many rows were taken from either end before it, and a claim is good while
// their sum is below n.  Every row is claimed once, and the meeting point settles where both kernels finish.
__device__ inline int64_t draw_front(unsigned long long *ticket, int64_t n, int64_t *slot)
{
    if (threadIdx.x == 0) {
        const unsigned long long old = atomicAdd(ticket, 1ull);
        const int64_t f = (int64_t)(old & 0xffffffffull), b = (int64_t)(old >> 32);
        *slot = f + b < n ? f : n;
    }
    __syncthreads();
    const int64_t r = *slot;
    __syncthreads();
    const int lo = __builtin_amdgcn_readfirstlane((int)(r & 0xffffffff));
    const int hi = __builtin_amdgcn_readfirstlane((int)(r >> 32));
    return ((int64_t)hi << 32) | (uint32_t)lo;
}

// Semiring operators of C = A @(reduce, mult) B.  The codes are the C ABI's.
enum { SR_PLUS = 0, SR_MIN = 1, SR_MAX = 2, SR_ANY = 3 };
__device__ inline double semiring_mult(int op, double a, double b)
{
    switch (op) {
    case 0: return a * b;
    case 1: return a;
    case 2: return b;
    case 3: return 1.0;
    case 4: return a + b;
    case 5: return a - b;
    case 6: return a < b ? a : b;
    case 7: return a > b ? a : b;
    default: return a / b;
    }
}
// Order-preserving map of a double onto an unsigned integer and back: min and
// max become integer atomics whose result does not depend on the order of the
// products, and an all-zero slot can stand for "nothing stored yet".
__device__ inline unsigned long long f64_key(double x)
{
    const unsigned long long u = (unsigned long long)__double_as_longlong(x);
    return (u >> 63) ? ~u : (u | 0x8000000000000000ull);
}
__device__ inline double key_f64(unsigned long long k)
{
    const unsigned long long u = (k >> 63) ? (k & 0x7fffffffffffffffull) : ~k;
    return __longlong_as_double((long long)u);
}
// One product of a semiring into an accumulator in LDS.  plus adds; min, max and any keep a 64-bit key and take the
// larger one, so the result does not depend on the order of the products: min the complement of the value's key,
// max the key, any the place (pa, q) of the product - pa counts the entries of the row of A from 1, q is the place
// in B - so that the product the reference's sequential loop reaches last wins.  An accumulator that received
// nothing is all-zero whatever the semiring.
__device__ __forceinline__ void semiring_lds_add(double *slot, int reduce_op, int mult_op, double a, double b, int pa,
                                                 int64_t q)
{
    unsigned long long *key = reinterpret_cast<unsigned long long *>(slot);
    if (reduce_op == SR_ANY) {
        __hip_atomic_fetch_max(key, ((unsigned long long)(uint32_t)pa << 32) | (unsigned long long)(uint32_t)q,
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    } else {
        const double e = semiring_mult(mult_op, a, b);
        if (reduce_op == SR_PLUS)
            __hip_atomic_fetch_add(slot, e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        else
            __hip_atomic_fetch_max(key, reduce_op == SR_MIN ? ~f64_key(e) : f64_key(e), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_WORKGROUP);
    }
}
// The value such an accumulator stands for (as = where the row of A begins).  max starts from 0, as the reference's
// accumulator does, and so never returns less.
__device__ __forceinline__ double semiring_lds_value(unsigned long long v, int reduce_op, int mult_op, int64_t as,
                                                     const double *__restrict__ Aval, const double *__restrict__ Bval)
{
    if (reduce_op == SR_PLUS)
        return __longlong_as_double((long long)v);
    if (reduce_op == SR_MIN)
        return key_f64(~v);
    if (reduce_op == SR_MAX)
        return v < f64_key(0.0) ? 0.0 : key_f64(v);
    return semiring_mult(mult_op, Aval[as + (int64_t)(v >> 32) - 1], Bval[(int64_t)(v & 0xffffffffull)]);
}
// Every kernel here carves its dynamic LDS into 32-bit words and fp64 regions (ds_add_f64 and 64-bit reads fault on
// an address that is not a multiple of 8): the array itself starts 16-byte aligned, and every fp64 region begins an
// even number of words into it - asserted where each layout is defined.
extern __shared__ __align__(16) uint32_t sg_dyn_lds[];
// Hash table of a masked product's mask row (see spgemm_numeric_kernel): values first (8-byte aligned), keys after.
constexpr int SG_HASH_LOG = 13, SG_HASH_SLOTS = 1 << SG_HASH_LOG;
static_assert((2 * SG_HASH_SLOTS) % 2 == 0 && SG_HASH_SLOTS % 2 == 0, "hash table: values at word 0, keys an even number of words in");
#ifndef COMET_SG_HASH_FILL
#define COMET_SG_HASH_FILL (SG_HASH_SLOTS * 3 / 4)
#endif
constexpr int SG_HASH_FILL = COMET_SG_HASH_FILL;          // longest mask row that goes into the table
constexpr size_t SG_HASH_LDS = (size_t)SG_HASH_SLOTS * (8 + 4);
// The first slot a column is looked for in.  (Keeping groups of 32 neighbouring columns together, so that the
// look-ups of a wavefront walking a sorted row fall into neighbouring LDS banks, was slower: 370 against 240 ms on
// A*A masked by A at R-MAT scale 20 - a miss that lands in such a group walks to its end.)
__device__ inline uint32_t sg_hash_slot(int j)
{
    return ((uint32_t)j * 2654435761u) >> (32 - SG_HASH_LOG);
}

// ---------------------------------------------------------------------------
// Symbolic phase.  Unmasked: set the bit of every reachable column, count the
// bits that were new.  Masked: the bitmap starts as the mask row; a product
// clears its bit, and the bits that were still set are the output entries.
// ---------------------------------------------------------------------------
template <bool BM_LDS, bool MASKED>
__global__ __launch_bounds__(SG_T) void spgemm_symbolic_kernel(
    int64_t nrows, const int64_t *__restrict__ Apos, const int32_t *__restrict__ Acrd,
    const int64_t *__restrict__ Bpos, const int32_t *__restrict__ Bcrd, const int64_t *__restrict__ Mpos,
    const int32_t *__restrict__ Mcrd, int logW, uint32_t *__restrict__ gbm, unsigned long long *ticket,
    RowList list, int64_t *__restrict__ rowcount)
{
    __shared__ int64_t row_slot;
    __shared__ int wave_cnt[SG_WAVES];
    uint32_t *bm;
    if constexpr (BM_LDS)
        bm = sg_dyn_lds;
    else
        bm = gbm + (size_t)blockIdx.x * (size_t)(SG_T * ((1 << logW) + 1));
    const BmAddr ad{logW};
    const int nwords = SG_T * ((1 << logW) + 1);
    if constexpr (BM_LDS) {
        for (int w = threadIdx.x; w < nwords; w += SG_T)
            bm[w] = 0;
    }
    __syncthreads();
    int64_t t_first, t_end;
    list_range(list, 2, &t_first, &t_end);
    int64_t t = draw_row(ticket, t_first, &row_slot);
    while (t < t_end) {
        const int64_t i = list.rows[t];       // rows outside the list keep the zero the host put there
        const int64_t as = Apos[i], ae = Apos[i + 1];
        int64_t ms = 0, me = 1;
        if constexpr (MASKED) {
            ms = Mpos[i];
            me = Mpos[i + 1];
        }
        const bool work = as != ae && ms != me;
        if (work) {
        if constexpr (MASKED) {
            for (int64_t t = ms + threadIdx.x; t < me; t += SG_T)
                atomicOr(&bm[ad.word(Mcrd[t])], ad.bit(Mcrd[t]));
            __syncthreads();
        }
        int count = 0;
        for_each_product<false>(as, ae, Acrd, nullptr, Bpos, Bcrd, [&](int j, int64_t, double, int64_t, int64_t) {
            const uint32_t b = ad.bit(j);
            if constexpr (MASKED) {
                const uint32_t old = atomicAnd(&bm[ad.word(j)], ~b);
                count += (old & b) ? 1 : 0;
            } else if constexpr (BM_LDS) {
                atomicOr(&bm[ad.word(j)], b);       // nothing comes back, so the walk never waits for LDS:
            } else {                                // the bits are counted when the bitmap is cleared
                const uint32_t old = atomicOr(&bm[ad.word(j)], b);
                count += (old & b) ? 0 : 1;
            }
        }, [&](sg_i4u j, int64_t, double, int64_t, int64_t) {
            // four consecutive entries of a sorted row: the bits that fall into one word go there together
            if constexpr (BM_LDS && !MASKED) {
                int w = ad.word(j.x);
                uint32_t b = ad.bit(j.x);
                const int js[3] = {j.y, j.z, j.w};
#pragma unroll
                for (int x = 0; x < 3; ++x) {
                    const int wx = ad.word(js[x]);
                    if (wx != w) {
                        atomicOr(&bm[w], b);
                        w = wx;
                        b = 0u;
                    }
                    b |= ad.bit(js[x]);
                }
                atomicOr(&bm[w], b);
            } else {
                const int js[4] = {j.x, j.y, j.z, j.w};
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const uint32_t b = ad.bit(js[x]);
                    if constexpr (MASKED) {
                        const uint32_t old = atomicAnd(&bm[ad.word(js[x])], ~b);
                        count += (old & b) ? 1 : 0;
                    } else {
                        const uint32_t old = atomicOr(&bm[ad.word(js[x])], b);
                        count += (old & b) ? 0 : 1;
                    }
                }
            }
        });
        if constexpr (BM_LDS && !MASKED) {
            __syncthreads();
            for (int w = threadIdx.x; w < nwords; w += SG_T) {
                count += __popc(bm[w]);
                bm[w] = 0;
            }
        }
        count = wave_sum_i32(count);
        if ((threadIdx.x & 63) == 0)
            wave_cnt[threadIdx.x >> 6] = count;
        __syncthreads();
        if (threadIdx.x == 0) {
            int total = 0;
            for (int w = 0; w < SG_WAVES; ++w)
                total += wave_cnt[w];
            rowcount[i] = total;
        }
        // leave the bitmap all-zero for the next row
        if constexpr (MASKED) {
            for (int64_t t = Mpos[i] + threadIdx.x; t < Mpos[i + 1]; t += SG_T)
                atomicAnd(&bm[ad.word(Mcrd[t])], 0u);
        } else if constexpr (!BM_LDS) {
            for_each_product<false>(as, ae, Acrd, nullptr, Bpos, Bcrd,
                                    [&](int j, int64_t, double, int64_t, int64_t) { atomicAnd(&bm[ad.word(j)], 0u); });
        }
        }   // work
        t = draw_row(ticket, t_first, &row_slot);     // its barriers also close this row's bitmap clean-up
    }
}

// ---------------------------------------------------------------------------
// Numeric phase for rows [row_begin,row_end).
// ---------------------------------------------------------------------------
// SEMI: any reduction/multiplication pair.  plus adds with the same fp64 atomic;
// min, max and any keep an integer key in the slab instead of a double and
// combine with an atomic max, so their results are independent of the order in
// which the products arrive: min stores the complement of the value's key, max
// the key itself (and, like the reference, never returns less than 0), any the
// position (p, q) of the product and so keeps the one a sequential traversal
// would reach last.  A slot is back to all-zero after extraction in every case.
template <bool BM_LDS, bool MASKED, bool SEMI>
__global__ __launch_bounds__(SG_T) void spgemm_numeric_kernel(
    int64_t row_begin, int64_t row_end, int64_t ncols, const int64_t *__restrict__ Apos,
    const int32_t *__restrict__ Acrd, const double *__restrict__ Aval, const int64_t *__restrict__ Bpos,
    const int32_t *__restrict__ Bcrd, const double *__restrict__ Bval, const int64_t *__restrict__ Mpos,
    const int32_t *__restrict__ Mcrd, int logW, uint32_t *__restrict__ gbm, uint32_t *__restrict__ gmask,
    double *__restrict__ slabs, unsigned long long *ticket, RowList list, int part,
    int reduce_op, int mult_op, const int64_t *__restrict__ Cpos,
    int32_t *__restrict__ Ccrd, double *__restrict__ Cval)
{
    __shared__ int64_t row_slot;
    __shared__ int wave_tot[SG_WAVES];
    // Two bitmaps: the columns of the output row (bm) and, for a masked product, the mask row (mbm).  One of
    // them fits LDS.  Unmasked, that is bm.  Masked, it is the mask: every product probes it, while only the
    // products that fall on a mask entry touch bm, which then lives in HBM with the slab and, like the slab,
    // is reached through L2 atomics only.
    constexpr bool OUT_LDS = BM_LDS && !MASKED, MASK_LDS = BM_LDS && MASKED;
    uint32_t *bm, *mbm = nullptr;
    if constexpr (OUT_LDS)
        bm = sg_dyn_lds;
    else
        bm = gbm + (size_t)blockIdx.x * (size_t)(SG_T * ((1 << logW) + 1));
    if constexpr (MASK_LDS)
        mbm = sg_dyn_lds;
    else if constexpr (MASKED)
        mbm = gmask + (size_t)blockIdx.x * (size_t)(SG_T * ((1 << logW) + 1));
    double *slab = slabs + (size_t)blockIdx.x * (size_t)ncols;
    const BmAddr ad{logW};
    const int W = 1 << logW;
    const int nwords = SG_T * ((1 << logW) + 1);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if constexpr (BM_LDS) {
        // the bitmap and, for a masked product, the hash table that shares its place
        const int lds_words = MASKED && nwords < (int)(SG_HASH_LDS / 4) ? (int)(SG_HASH_LDS / 4) : nwords;
        for (int w = threadIdx.x; w < lds_words; w += SG_T)
            sg_dyn_lds[w] = 0;
    }
    __syncthreads();
    const int64_t out0 = Cpos[row_begin];
    int64_t t_first, t_end;
    list_range(list, part, &t_first, &t_end);      // rows with many products are left to spgemm_numeric_dense_kernel
    int64_t t = draw_row(ticket, t_first, &row_slot);
    while (t < t_end) {
        const int64_t i = row_begin + list.rows[t];
        const int64_t as = Apos[i], ae = Apos[i + 1];
        const int64_t ob = Cpos[i], oe = Cpos[i + 1];
        bool hashed = false;
        if constexpr (MASK_LDS)
            hashed = __builtin_amdgcn_readfirstlane((int)(Mpos[i + 1] - Mpos[i] <= SG_HASH_FILL)) != 0;
        if (as != ae && ob != oe && hashed) {
            // A mask row of at most SG_HASH_FILL entries (nearly every row) goes into a hash table in LDS, column
            // -> slot, and the slot holds the value: a product probes the table (one LDS read for the 96 % that
            // miss), a product that falls on a mask entry adds into the slot with an LDS atomic, and nothing of
            // the row touches the L2.  A slot's key is column + 1, bit 31 says that a product has arrived.
            uint32_t *hkey = sg_dyn_lds + 2 * SG_HASH_SLOTS;
            double *hval = reinterpret_cast<double *>(sg_dyn_lds);
            unsigned long long *hbits = reinterpret_cast<unsigned long long *>(sg_dyn_lds);
            const auto slot_of = [&](int j) -> int {          // the slot that holds column j, or -1
                uint32_t sl = sg_hash_slot(j);
                for (;;) {
                    const uint32_t k = hkey[sl];
                    if ((k & 0x7fffffffu) == (uint32_t)j + 1u)
                        return (int)sl;
                    if (k == 0u)
                        return -1;
                    sl = (sl + 1) & (SG_HASH_SLOTS - 1);
                }
            };
            const int64_t ms = Mpos[i], mlen = Mpos[i + 1] - ms;
            for (int64_t e = ms + threadIdx.x; e < ms + mlen; e += SG_T) {
                const uint32_t key = (uint32_t)Mcrd[e] + 1u;
                uint32_t sl = sg_hash_slot(Mcrd[e]);
                for (;;) {
                    const uint32_t old = atomicCAS(&hkey[sl], 0u, key);
                    if (old == 0u || old == key)
                        break;
                    sl = (sl + 1) & (SG_HASH_SLOTS - 1);
                }
            }
            __syncthreads();
            const auto first_slot = [](int j) { return sg_hash_slot(j); };
            for_each_product_probed<true>(as, ae, Acrd, Aval, Bpos, Bcrd, [&](int j) { return hkey[first_slot(j)]; },
                                          [&](int j, int64_t q, uint32_t k0) {
                // k0 = the key in the column's first slot: nearly always that settles it
                MaskHit h{-1, 0.0};
                if (k0 != 0u)
                    h.at = (k0 & 0x7fffffffu) == (uint32_t)j + 1u ? (int)first_slot(j) : slot_of(j);
                if (h.at >= 0 && !(SEMI && reduce_op == SR_ANY))
                    h.b = Bval[q];
                return h;
            }, [&](int j, int64_t q, double a, int64_t p, int64_t bs, MaskHit h) {
                const int sl = h.at;
                if (sl < 0)
                    return;
                if (!(hkey[sl] >> 31))
                    atomicOr(&hkey[sl], 0x80000000u);
                if constexpr (SEMI) {
                    if (reduce_op == SR_ANY) {
                        const unsigned long long key = ((unsigned long long)(p - as + 1) << 32) | (unsigned long long)(q - bs);
                        __hip_atomic_fetch_max(&hbits[sl], key, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    } else {
                        const double e = semiring_mult(mult_op, a, h.b);
                        if (reduce_op == SR_PLUS)
                            __hip_atomic_fetch_add(&hval[sl], e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                        else
                            __hip_atomic_fetch_max(&hbits[sl], reduce_op == SR_MIN ? ~f64_key(e) : f64_key(e),
                                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    }
                } else {
                    __hip_atomic_fetch_add(&hval[sl], a * h.b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
            });
            __syncthreads();
            // the mask row is sorted: thread t takes a run of its entries, counts the ones a product reached, and
            // after a prefix sum over the workgroup writes them in place
            const int64_t per = (mlen + SG_T - 1) / SG_T;
            const int64_t e0 = ms + (int64_t)threadIdx.x * per;
            const int64_t e1 = e0 + per < ms + mlen ? e0 + per : ms + mlen;
            int mine = 0;
            for (int64_t e = e0; e < e1; ++e) {
                const int j = Mcrd[e];
                if (e > ms && Mcrd[e - 1] == j)
                    continue;          // a column stored twice in the mask row is one output entry
                mine += (int)(hkey[slot_of(j)] >> 31);
            }
            const int inc = wave_inclusive_scan(mine);
            if (lane == 63)
                wave_tot[wave] = inc;
            __syncthreads();
            int64_t off = ob - out0 + (inc - mine);
            for (int w = 0; w < wave; ++w)
                off += wave_tot[w];
            for (int64_t e = e0; e < e1; ++e) {
                const int j = Mcrd[e];
                if (e > ms && Mcrd[e - 1] == j)
                    continue;
                const int sl = slot_of(j);
                if (!(hkey[sl] >> 31))
                    continue;
                Ccrd[off] = j;
                double out = hval[sl];
                if (SEMI && reduce_op != SR_PLUS) {
                    const unsigned long long v = hbits[sl];
                    if (reduce_op == SR_MIN) {
                        out = key_f64(~v);
                    } else if (reduce_op == SR_MAX) {
                        out = v < f64_key(0.0) ? 0.0 : key_f64(v);
                    } else {
                        const int64_t pp = as + (int64_t)(v >> 32) - 1;
                        const int64_t qq = Bpos[Acrd[pp]] + (int64_t)(v & 0xffffffffull);
                        out = semiring_mult(mult_op, Aval[pp], Bval[qq]);
                    }
                }
                Cval[off] = out;
                ++off;
            }
            __syncthreads();           // everybody has found its slots: now they are emptied (keys last used above)
            for (int sl = threadIdx.x; sl < SG_HASH_SLOTS; sl += SG_T)
                if (hkey[sl]) {
                    hkey[sl] = 0u;
                    hbits[sl] = 0ull;
                }
        }
        if (as != ae && ob != oe && !hashed) {
        if constexpr (MASKED) {
            for (int64_t t = Mpos[i] + threadIdx.x; t < Mpos[i + 1]; t += SG_T)
                atomicOr(&mbm[ad.word(Mcrd[t])], ad.bit(Mcrd[t]));
            __syncthreads();
        }
        for_each_product_probed<true>(as, ae, Acrd, Aval, Bpos, Bcrd, [&](int j) {
            if constexpr (MASK_LDS)
                return mbm[ad.word(j)];      // the mask row was set before the barrier above and does not change
            else
                return 0u;
        }, [&](int j, int64_t q, uint32_t mword) {
            MaskHit h{0, 0.0};
            if constexpr (MASK_LDS)
                h.at = (mword & ad.bit(j)) ? 0 : -1;
            else if constexpr (MASKED)
                h.at = (atomicOr(&mbm[ad.word(j)], 0u) & ad.bit(j)) ? 0 : -1;
            if (h.at >= 0 && !(SEMI && reduce_op == SR_ANY))
                h.b = Bval[q];
            return h;
        }, [&](int j, int64_t q, double a, int64_t p, int64_t bs, MaskHit h) {
            if (h.at < 0)
                return;
            const int w = ad.word(j);
            const uint32_t b = ad.bit(j);
            atomicOr(&bm[w], b);
            if constexpr (SEMI) {
                unsigned long long *slot = (unsigned long long *)&slab[j];
                if (reduce_op == SR_ANY) {
                    const unsigned long long key = ((unsigned long long)(p - as + 1) << 32) | (unsigned long long)(q - bs);
                    __hip_atomic_fetch_max(slot, key, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                } else {
                    const double e = semiring_mult(mult_op, a, h.b);
                    if (reduce_op == SR_PLUS)
                        __hip_atomic_fetch_add(&slab[j], e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    else
                        __hip_atomic_fetch_max(slot, reduce_op == SR_MIN ? ~f64_key(e) : f64_key(e),
                                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
            } else {
                __hip_atomic_fetch_add(&slab[j], a * h.b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
        });
        __syncthreads();
        if constexpr (MASK_LDS) {
            // (rows whose mask row fits the hash table never come here: see below)
            // The output row is a subset of the mask row: walk that (it is sorted) instead of the bitmap.  Thread t
            // takes a run of consecutive mask entries, counts those whose bit a product has set, and after a prefix
            // sum over the workgroup writes them in place; value and bit are fetched and cleared on the way.
            const int64_t ms = Mpos[i], mlen = Mpos[i + 1] - ms;
            const int64_t per = (mlen + SG_T - 1) / SG_T;
            const int64_t e0 = ms + (int64_t)threadIdx.x * per;
            const int64_t e1 = e0 + per < ms + mlen ? e0 + per : ms + mlen;
            int mine = 0;
            for (int64_t e = e0; e < e1; ++e) {
                const int j = Mcrd[e];
                if (e > ms && Mcrd[e - 1] == j)
                    continue;          // a column stored twice in the mask row is one output entry
                mine += (atomicOr(&bm[ad.word(j)], 0u) & ad.bit(j)) ? 1 : 0;
            }
            int inc = wave_inclusive_scan(mine);
            if (lane == 63)
                wave_tot[wave] = inc;
            __syncthreads();           // also: every bit has been read before the first one is cleared below
            int64_t off = ob - out0 + (inc - mine);
            for (int w = 0; w < wave; ++w)
                off += wave_tot[w];
            for (int64_t e = e0; e < e1; ++e) {
                const int j = Mcrd[e];
                if ((e > ms && Mcrd[e - 1] == j) || !(atomicOr(&bm[ad.word(j)], 0u) & ad.bit(j)))
                    continue;
                Ccrd[off] = j;
                if (SEMI && reduce_op != SR_PLUS) {
                    const unsigned long long v = __hip_atomic_exchange((unsigned long long *)&slab[j], 0ull,
                                                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    double out;
                    if (reduce_op == SR_MIN) {
                        out = key_f64(~v);
                    } else if (reduce_op == SR_MAX) {
                        out = v < f64_key(0.0) ? 0.0 : key_f64(v);
                    } else {
                        const int64_t pp = as + (int64_t)(v >> 32) - 1;
                        const int64_t qq = Bpos[Acrd[pp]] + (int64_t)(v & 0xffffffffull);
                        out = semiring_mult(mult_op, Aval[pp], Bval[qq]);
                    }
                    Cval[off] = out;
                } else {
                    Cval[off] = __hip_atomic_exchange(&slab[j], 0.0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
                ++off;
            }
            __syncthreads();           // all reads of the bits are done
            for (int64_t e = e0; e < e1; ++e) {
                const int j = Mcrd[e];
                atomicAnd(&bm[ad.word(j)], ~ad.bit(j));
                atomicAnd(&mbm[ad.word(j)], 0u);
            }
        } else {
        // extraction: my words hold my columns in ascending order
        int mine = 0;
        for (int k = 0; k < W; ++k)
            mine += __popc(OUT_LDS ? bm[threadIdx.x * (W + 1) + k] : atomicOr(&bm[threadIdx.x * (W + 1) + k], 0u));
        int inc = mine;
        for (int d = 1; d < 64; d <<= 1) {
            const int o = __shfl_up(inc, d, 64);
            if (lane >= d)
                inc += o;
        }
        if (lane == 63)
            wave_tot[wave] = inc;
        __syncthreads();
        int64_t off = ob - out0 + (inc - mine);
        for (int w = 0; w < wave; ++w)
            off += wave_tot[w];
        for (int k = 0; k < W; ++k) {
            uint32_t word;
            if constexpr (OUT_LDS) {
                word = bm[threadIdx.x * (W + 1) + k];
                bm[threadIdx.x * (W + 1) + k] = 0;
            } else {
                word = atomicAnd(&bm[threadIdx.x * (W + 1) + k], 0u);
            }
            const int jbase = (((int)threadIdx.x << logW) + k) << 5;
            while (word) {
                const int b = __ffs(word) - 1;
                word &= word - 1;
                const int j = jbase + b;
                Ccrd[off] = j;
                if (SEMI && reduce_op != SR_PLUS) {
                    const unsigned long long v = __hip_atomic_exchange((unsigned long long *)&slab[j], 0ull,
                                                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    double out;
                    if (reduce_op == SR_MIN) {
                        out = key_f64(~v);
                    } else if (reduce_op == SR_MAX) {
                        out = v < f64_key(0.0) ? 0.0 : key_f64(v);
                    } else {
                        const int64_t pp = as + (int64_t)(v >> 32) - 1;
                        const int64_t qq = Bpos[Acrd[pp]] + (int64_t)(v & 0xffffffffull);
                        out = semiring_mult(mult_op, Aval[pp], Bval[qq]);
                    }
                    Cval[off] = out;
                } else {
                    Cval[off] = __hip_atomic_exchange(&slab[j], 0.0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
                ++off;
            }
        }
        if constexpr (MASKED) {
            for (int64_t t = Mpos[i] + threadIdx.x; t < Mpos[i + 1]; t += SG_T)
                atomicAnd(&mbm[ad.word(Mcrd[t])], 0u);
        }
        }   // extraction over the bitmap
        }   // row with output
        t = draw_row(ticket, t_first, &row_slot);     // its barriers also close this row's clean-up
    }
}

// ---------------------------------------------------------------------------
// Numeric phase for rows with many products: the L2 performs only ~20 G atomic
// line operations per second, so the slab path above costs one of those per
// product.  Here a row is swept in blocks of 16384 columns whose accumulators
// (128 KiB of doubles) and bitmap live in LDS; the products of one block are
// found through the per-row block pointers of B's plan.  Blocks are visited in
// ascending order and each is emitted in bitmap order, so the row still comes
// out sorted.
// ---------------------------------------------------------------------------
constexpr int SG_CB_LOG = 14;
constexpr int SG_CB = 1 << SG_CB_LOG;                                 // columns per block
typedef uint16_t emit_t;                                              // a column of the block being written out
constexpr int SG_EMIT = 8192;                                         // entries written out per turn of the emit
constexpr size_t SG_DENSE_LDS = (size_t)SG_CB * 8 + (size_t)SG_CB / 8 + (size_t)SG_EMIT * sizeof(emit_t) +
                                2 * (size_t)SG_CB / 8;               // accumulators, bitmap, list of the columns being
                                                                      // written out, the mask row's bits (two blocks)
// the accumulators (fp64) come first; what follows them is 32- and 16-bit data and starts on a word
static_assert(((size_t)SG_CB * 8) % 8 == 0 && ((size_t)SG_CB / 8) % 4 == 0 && ((size_t)SG_EMIT * sizeof(emit_t)) % 4 == 0,
              "the one-block kernel's LDS regions are aligned for their types");

// products[i - row_begin] = sum over k in A_i of nnz(B_k); one wavefront per row.  With Tpos (the dot-product form of
// a masked product, where row i's pairs k are shared out by which of the two lists is longer) only the k whose row
// of B is shorter than row i of T (strict) or not longer (otherwise), and that lie in [xlo, xhi), count.
__global__ __launch_bounds__(256) void spgemm_row_products(int64_t row_begin, int64_t row_end,
                                                           const int64_t *__restrict__ Apos,
                                                           const int32_t *__restrict__ Acrd,
                                                           const int64_t *__restrict__ Bpos,
                                                           int64_t *__restrict__ products,
                                                           const int64_t *__restrict__ Tpos = nullptr, int strict = 0,
                                                           int64_t xlo = 0, int64_t xhi = 0)
{
    const int64_t i = row_begin + (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= row_end)
        return;
    const int lane = threadIdx.x & 63;
    const int64_t tlen = Tpos ? Tpos[i + 1] - Tpos[i] : 0;
    int64_t s = 0;
    for (int64_t p = Apos[i] + lane; p < Apos[i + 1]; p += 64) {
        const int k = Acrd[p];
        const int64_t len = Bpos[k + 1] - Bpos[k];
        if (!Tpos || ((strict ? len < tlen : len <= tlen) && k >= xlo && k < xhi))
            s += len;
    }
    for (int d = 32; d > 0; d >>= 1)
        s += __shfl_down(s, d, 64);
    if (lane == 0)
        products[i - row_begin] = s;
}

// blkptr[k * (nblk + 1) + cb] = position in crd/val of the first entry of row k whose column is >= cb * SG_CB
// (cb = nblk gives the end of the row): the slice of row k inside block cb is one 16-byte load away.
// crd16[q] = the column of entry q inside its block of SG_CB columns
__global__ void spgemm_block_columns(int64_t nnz, const int32_t *__restrict__ crd, uint16_t *__restrict__ crd16)
{
    const int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (q < nnz)
        crd16[q] = (uint16_t)(crd[q] & (SG_CB - 1));
}

__global__ void spgemm_block_pointers(int64_t nrows, const int64_t *__restrict__ pos,
                                      const int32_t *__restrict__ crd, int nblk, int64_t *__restrict__ blkptr)
{
    const int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= nrows)
        return;
    const int64_t s = pos[k], e = pos[k + 1];
    int64_t *out = blkptr + k * (nblk + 1);
    int64_t lo = s;
    out[0] = s;
    for (int cb = 1; cb <= nblk; ++cb) {
        const int64_t bound = (int64_t)cb << SG_CB_LOG;
        int64_t hi = e;
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (crd[mid] < bound)
                lo = mid + 1;
            else
                hi = mid;
        }
        out[cb] = lo;
    }
}

// One barrier tells every wavefront of the workgroup whether any of them had work in this visit.  The answer is
// made scalar, so that a branch on it is uniform (the branches taken on it hold barriers).  Three flags take
// turns: a wavefront may be a whole visit ahead of the slowest one, which is still to read this visit's flag
// when the fast one raises the next; the flag of the visit after that is cleared here, before the barrier,
// when everybody has long read its last use (they all came through the previous visit's barrier since).
__device__ __forceinline__ int visit_flag(int *flags, int visit, int touched, int lane)
{
    if (threadIdx.x == 0)
        flags[visit == 2 ? 0 : visit + 1] = 0;
    if (touched && lane == 0)
        flags[visit] = 1;
    lds_barrier();
    return __builtin_amdgcn_readfirstlane(flags[visit]);
}

// Visits the products of one slice per lane: f(j, a, b, pa, q) for the entries [lo, hi) of a row of B (the part of
// it inside the column block or blocks being swept), j the column, a the entry of A (and pa the tag the caller
// gave it: its place in the row of A, which only the `any` semiring needs), b the entry of B (0 without VALUES,
// when the value array is not read) and q its place in B.  Returns whether this wavefront had anything to visit.

#ifndef COMET_SG_SHORT
#define COMET_SG_SHORT 32
#endif
constexpr int SG_SHORT = COMET_SG_SHORT;          // slices shorter than this are laid end to end, the others take turns of their own
constexpr int SG_SHORT_LOADS = 2;                 // entries of the short slices per lane and batch
constexpr int SG_LONG_LOADS = 4;                  // entries of a long slice per lane and turn

// One turn of a wavefront over a slice that starts at entry s of B and has len entries: lane l visits the
// entries o + 64 x < len, x < SG_LONG_LOADS (o = l for the first turn of a slice).  All loads are issued before
// the first visit, and a load that no lane needs is skipped.
// The columns of B come as 32-bit numbers or (COL = uint16_t) as the 16-bit numbers inside their block of SG_CB
// columns that the right-hand operand's plan keeps for the kernel that takes one block per visit: a third of the
// bytes of an entry it only needs the column of.
typedef unsigned short sg_h4u __attribute__((ext_vector_type(4), aligned(2)));
typedef double sg_d2u __attribute__((ext_vector_type(2), aligned(8)));
template <typename COL>
struct SgCol4;
template <>
struct SgCol4<int32_t> {
    typedef sg_i4u type;
};
template <>
struct SgCol4<uint16_t> {
    typedef sg_h4u type;
};

template <bool VALUES, typename COL, typename F>
__device__ __forceinline__ void turn_of_slice(int64_t s, int64_t o, int64_t len, double at, int pt,
                                              const COL *__restrict__ Bcrd, const double *__restrict__ Bval, F f)
{
    int64_t q[SG_LONG_LOADS];
    bool ok[SG_LONG_LOADS];
#pragma unroll
    for (int x = 0; x < SG_LONG_LOADS; ++x) {
        ok[x] = o + 64 * x < len;
        q[x] = ok[x] ? s + o + 64 * x : 0;
    }
    int j[SG_LONG_LOADS];
    double v[SG_LONG_LOADS];
#pragma unroll
    for (int x = 0; x < SG_LONG_LOADS; ++x)
        j[x] = ok[x] ? (int)Bcrd[q[x]] : 0;
#pragma unroll
    for (int x = 0; x < SG_LONG_LOADS; ++x)
        v[x] = VALUES && ok[x] ? Bval[q[x]] : 0.0;
#pragma unroll
    for (int x = 0; x < SG_LONG_LOADS; ++x)
        if (ok[x])
            f(j[x], at, v[x], pt, q[x]);
}

// A turn in which every lane has all its entries, the lane taking SG_LONG_LOADS consecutive ones (see the full turns of
// for_each_in_slices): f4(j, a, v0, v1, pa, q) for the entries q .. q + 3.
template <bool VALUES, typename COL, typename F4>
__device__ __forceinline__ void full_turn_of_slice(int64_t s, int lane, double at, int pt, const COL *__restrict__ Bcrd,
                                                   const double *__restrict__ Bval, F4 f4)
{
    typedef typename SgCol4<COL>::type col4;
    const int64_t c = s + 4 * (int64_t)lane;
    const col4 j = *reinterpret_cast<const col4 *>(Bcrd + c);
    sg_d2u v0 = {0.0, 0.0}, v1 = {0.0, 0.0};
    if constexpr (VALUES) {
        v0 = *reinterpret_cast<const sg_d2u *>(Bval + c);
        v1 = *reinterpret_cast<const sg_d2u *>(Bval + c + 2);
    }
    f4(j, at, v0, v1, pt, c);
}

struct SgOneByOne {};          // in place of f4: the four entries of a lane in a full turn go through f one by one
template <bool VALUES, typename COL, typename F, typename F4 = SgOneByOne>
__device__ __forceinline__ int for_each_in_slices(int64_t lo, int64_t hi, double a, int pa, int lane,
                                                  const COL *__restrict__ Bcrd,
                                                  const double *__restrict__ Bval, F f, F4 f4 = F4())
{
    typedef typename SgCol4<COL>::type col4;
    // f4(j, a, v0, v1, pa, q): the four consecutive entries q .. q + 3 of one row of B, columns j, values v0.x, v0.y,
    // v1.x, v1.y
    const auto four = [&](col4 j, double at, auto v0, auto v1, int pt, int64_t c) {
        if constexpr (std::is_same<F4, SgOneByOne>::value) {
            f((int)j.x, at, v0.x, pt, c);
            f((int)j.y, at, v0.y, pt, c + 1);
            f((int)j.z, at, v1.x, pt, c + 2);
            f((int)j.w, at, v1.y, pt, c + 3);
        } else {
            f4(j, at, v0, v1, pt, c);
        }
    };
    // Long slices take the whole wavefront, one at a time; short ones (a slice of one block often holds a
    // dozen entries) are laid end to end and dealt to the lanes entry by entry (below).  A wavefront runs its
    // turns one after the other (there is room for one workgroup per CU, so nobody else hides the latency), and
    // a turn costs about one trip to memory: so every turn issues all of its loads before the first LDS
    // operation waits for one, and a load that no lane needs is skipped.  Measured on A*A of an R-MAT
    // graph of scale 20: two loads per lane and turn of a long slice instead of four, +18 % time in this
    // kernel, eight +2 %; two long slices per turn, +2..8 %; slices of up to 4 or 8 entries left to their own
    // lane (64 slices per turn, but every lane a cache line of its own), +4..6 %; the short slices one to a
    // 16-lane quarter, four at a time, +1.7 % (up to 64 or 128 entries that way, +1..5 % more); laid end to
    // end up to 128 or 256 entries instead of 32, +6 % and +22 %.
    unsigned long long big = __ballot(hi - lo >= SG_SHORT);
    unsigned long long todo = __ballot(lo < hi && hi - lo < SG_SHORT);
    const int touched = (big | todo) != 0;
    while (big) {               // one long slice per turn, up to SG_LONG_LOADS entries of it per lane
        const int t = __builtin_ctzll(big);
        big &= big - 1;
        const int64_t s = readlane_i64(lo, t), len = readlane_i64(hi, t) - s;
        const double at = readlane_d(a, t);
        const int pt = __builtin_amdgcn_readlane(pa, t);
        int64_t o = lane;
        if (len >= 64 * SG_LONG_LOADS) {
            // turns in which every lane has all its entries run without predicates, and the loads of the next
            // such turn are in flight while this one's products go into LDS
            // In a full turn a lane takes SG_LONG_LOADS consecutive entries: one 16-byte load of columns and two of
            // values per lane instead of four loads of each, a stride of 64 entries apart.  (Entries of B lie at any
            // 4- and 8-byte boundary: the loads are declared unaligned.)
            static_assert(SG_LONG_LOADS == 4, "a lane's entries of a full turn are one 16-byte load of columns");
            int64_t c = s + 4 * (int64_t)lane;          // this lane's first entry of the turn
            col4 j = *reinterpret_cast<const col4 *>(Bcrd + c);
            sg_d2u v0 = {0.0, 0.0}, v1 = {0.0, 0.0};
            if constexpr (VALUES) {
                v0 = *reinterpret_cast<const sg_d2u *>(Bval + c);
                v1 = *reinterpret_cast<const sg_d2u *>(Bval + c + 2);
            }
            int64_t done = 0;
            for (int64_t full = 64 * SG_LONG_LOADS; full + 64 * SG_LONG_LOADS <= len; full += 64 * SG_LONG_LOADS) {
                const int64_t cn = c + 64 * SG_LONG_LOADS;
                const col4 jn = *reinterpret_cast<const col4 *>(Bcrd + cn);
                sg_d2u v0n = {0.0, 0.0}, v1n = {0.0, 0.0};
                if constexpr (VALUES) {
                    v0n = *reinterpret_cast<const sg_d2u *>(Bval + cn);
                    v1n = *reinterpret_cast<const sg_d2u *>(Bval + cn + 2);
                }
                four(j, at, v0, v1, pt, c);
                j = jn;
                v0 = v0n;
                v1 = v1n;
                c = cn;
                done += 64 * SG_LONG_LOADS;
            }
            four(j, at, v0, v1, pt, c);
            done += 64 * SG_LONG_LOADS;
            o += done;
        }
        if (o < len)
            turn_of_slice<VALUES, COL>(s, o, len, at, pt, Bcrd, Bval, f);
    }
    // The short slices are laid end to end and dealt to the lanes entry by entry, 64 at a time, so that every load
    // and every LDS operation has all its lanes (a quarter-wavefront per slice left two thirds of them idle: a
    // slice of one block holds a dozen entries).  The lane that holds the slice an entry belongs to is found by
    // bisection over the running sum of the slices' lengths.
    if (todo) {
        const int mylen = (todo >> lane) & 1ull ? (int)(hi - lo) : 0;
        const int upto = wave_inclusive_scan(mylen);           // entries of the short slices of lanes 0..lane
        const int total = __builtin_amdgcn_readlane(upto, 63);
        // the entries e0 + 64 x + lane: where they lie in B, whose they are, and their loads
        const auto fetch = [&](int e0, bool *ok, int64_t *q, double *at, int *pt, int *j, double *v) {
#pragma unroll
            for (int x = 0; x < SG_SHORT_LOADS; ++x) {
                const int e = e0 + 64 * x + lane;
                ok[x] = e < total;
                int l = 0, h = 63;                  // the first lane whose running sum exceeds e
#pragma unroll
                for (int step = 0; step < 6; ++step) {
                    const int mid = (l + h) >> 1;
                    const bool right = __shfl(upto, mid, 64) <= e;
                    l = right ? mid + 1 : l;
                    h = right ? h : mid;
                }
                const int t = ok[x] ? l : lane;
                const int before = __shfl(upto - mylen, t, 64);
                const int64_t s = ((int64_t)__shfl((int)(lo >> 32), t, 64) << 32) |
                                  (uint32_t)__shfl((int)(lo & 0xffffffff), t, 64);
                q[x] = ok[x] ? s + (e - before) : 0;
                at[x] = __hiloint2double(__shfl(__double2hiint(a), t, 64), __shfl(__double2loint(a), t, 64));
                pt[x] = __shfl(pa, t, 64);
            }
#pragma unroll
            for (int x = 0; x < SG_SHORT_LOADS; ++x)
                j[x] = (ok[x] ? (int)Bcrd[q[x]] : 0);
#pragma unroll
            for (int x = 0; x < SG_SHORT_LOADS; ++x)
                v[x] = (VALUES && ok[x] ? Bval[q[x]] : 0.0);
        };
        bool ok[SG_SHORT_LOADS];
        int64_t q[SG_SHORT_LOADS];
        double at[SG_SHORT_LOADS], v[SG_SHORT_LOADS];
        int pt[SG_SHORT_LOADS], j[SG_SHORT_LOADS];
        fetch(0, ok, q, at, pt, j, v);
        for (int e0 = 0; e0 < total; e0 += 64 * SG_SHORT_LOADS) {
            // the next batch's loads are in flight while this one's products go into LDS
            bool okn[SG_SHORT_LOADS];
            int64_t qn[SG_SHORT_LOADS];
            double atn[SG_SHORT_LOADS], vn[SG_SHORT_LOADS];
            int ptn[SG_SHORT_LOADS], jn[SG_SHORT_LOADS];
            const bool more = e0 + 64 * SG_SHORT_LOADS < total;
            if (more)
                fetch(e0 + 64 * SG_SHORT_LOADS, okn, qn, atn, ptn, jn, vn);
#pragma unroll
            for (int x = 0; x < SG_SHORT_LOADS; ++x) {
                if (ok[x]) {
                    f(j[x], at[x], v[x], pt[x], q[x]);
                }
            }
            if (more) {
#pragma unroll
                for (int x = 0; x < SG_SHORT_LOADS; ++x) {
                    ok[x] = okn[x];
                    q[x] = qn[x];
                    at[x] = atn[x];
                    v[x] = vn[x];
                    pt[x] = ptn[x];
                    j[x] = jn[x];
                }
            }
        }
    }
    return touched;
}

// One product a * b for column j of the block that begins at column col0 (j counts from there with 16-bit columns):
// its bit is set and it is added to the column's accumulator in LDS.
template <bool SEMI, typename COL>
__device__ __forceinline__ void dense_add(double *acc, uint32_t *bm, int col0, int j, double a, double b, int pa,
                                          int64_t q, int reduce_op, int mult_op)
{
    if constexpr (sizeof(COL) == 4)
        j -= col0;
    atomicOr(&bm[j >> 5], 1u << (j & 31));
    if constexpr (SEMI)
        semiring_lds_add(&acc[j], reduce_op, mult_op, a, b, pa, q);
    else
        __hip_atomic_fetch_add(&acc[j], a * b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
// Four consecutive entries of a row of B at once (columns ascending): the bits that fall into one word of the bitmap
// go there together - lanes that walk a dense slice otherwise pile up on that word, four times each.
template <bool SEMI, typename COL, typename J4, typename V2>
__device__ __forceinline__ void dense_add4(double *acc, uint32_t *bm, int col0, J4 j4, double a, V2 v0, V2 v1, int pa,
                                           int64_t q, int reduce_op, int mult_op)
{
    int j[4] = {(int)j4.x, (int)j4.y, (int)j4.z, (int)j4.w};
    const double b[4] = {v0.x, v0.y, v1.x, v1.y};
    if constexpr (sizeof(COL) == 4) {
#pragma unroll
        for (int x = 0; x < 4; ++x)
            j[x] -= col0;
    }
    int w = j[0] >> 5;
    uint32_t bits = 1u << (j[0] & 31);
#pragma unroll
    for (int x = 1; x < 4; ++x) {
        if ((j[x] >> 5) != w) {
            atomicOr(&bm[w], bits);
            w = j[x] >> 5;
            bits = 0u;
        }
        bits |= 1u << (j[x] & 31);
    }
    atomicOr(&bm[w], bits);
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        if constexpr (SEMI)
            semiring_lds_add(&acc[j[x]], reduce_op, mult_op, a, b[x], pa, q + x);
        else
            __hip_atomic_fetch_add(&acc[j[x]], a * b[x], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
}
// the block's value of column j, which is cleared (as: where the row of A begins, for the semirings that keep places)
template <bool SEMI>
__device__ __forceinline__ double dense_take(double *acc, int j, int reduce_op, int mult_op, int64_t as,
                                             const double *__restrict__ Aval, const double *__restrict__ Bval)
{
    double out;
    if constexpr (SEMI)
        out = semiring_lds_value(reinterpret_cast<unsigned long long *>(acc)[j], reduce_op, mult_op, as, Aval, Bval);
    else
        out = acc[j];
    acc[j] = 0.0;
    return out;
}

// Writes out the block of SG_CB columns a workgroup holds in LDS (bitmap bm, accumulators read and cleared through
// take) as sorted entries of C and leaves the bitmap clean; returns how many.  place(total), which every thread
// calls once the number of entries is known, says where in Ccrd / Cval the first of them goes.  With MASKED the
// columns that are not set in mb are dropped and mb is cleared as well.
template <bool MASKED, typename TAKE, typename PLACE>
__device__ __forceinline__ int dense_emit_block(uint32_t *bm, uint32_t *mb, double *acc, emit_t *emit_col,
                                                int *wave_tot, int lane, int wave, int col0,
                                                int32_t *__restrict__ Ccrd, double *__restrict__ Cval, TAKE take,
                                                PLACE place)
{
    // Thread t owns the columns [8t, 8t + 8) and [8192 + 8t, 8192 + 8t + 8): one byte from each half of the bitmap,
    // so that the dense low columns of a half (the columns of a power-law graph thin out with the number of set
    // bits of the id) are spread over all the wavefronts.  The counts of the two bytes are scanned together,
    // packed into one word.
    static_assert(SG_T * 16 == SG_CB && SG_WAVES <= 64, "one byte of each half of the bitmap per thread");
    const uint8_t *bm8 = reinterpret_cast<const uint8_t *>(bm);
    uint32_t bits_a = bm8[threadIdx.x], bits_b = bm8[SG_CB / 16 + threadIdx.x];
    const int jbase = (int)threadIdx.x << 3;
    if constexpr (MASKED) {          // columns outside the mask row are dropped here
        const uint8_t *mb8 = reinterpret_cast<const uint8_t *>(mb);
        const uint32_t keep_a = mb8[threadIdx.x], keep_b = mb8[SG_CB / 16 + threadIdx.x];
        for (uint32_t w = bits_a & ~keep_a; w; w &= w - 1)
            acc[jbase + __ffs(w) - 1] = 0.0;
        for (uint32_t w = bits_b & ~keep_b; w; w &= w - 1)
            acc[SG_CB / 2 + jbase + __ffs(w) - 1] = 0.0;
        bits_a &= keep_a;
        bits_b &= keep_b;
    }
    const int mine = __popc(bits_a) | (__popc(bits_b) << 16);
    const int inc = wave_inclusive_scan(mine);
    if (lane == 63)
        wave_tot[wave] = inc;
    lds_barrier();
    const int tots = wave_inclusive_scan(lane < SG_WAVES ? wave_tot[lane] : 0);
    const int all = __builtin_amdgcn_readlane(tots, SG_WAVES - 1);
    const int before = (wave ? __builtin_amdgcn_readlane(tots, wave - 1) : 0) + inc - mine;
    const int total_a = all & 0xffff, total = total_a + (all >> 16);
    const int first_a = before & 0xffff, first_b = total_a + (before >> 16);
    const int64_t off = place(total);
    if (threadIdx.x < SG_CB / 32) {    // everybody has read its bytes: the bitmap is clean for the next block,
        bm[threadIdx.x] = 0;           // which nobody enters before the barrier below
        if constexpr (MASKED)
            mb[threadIdx.x] = 0;
    }
    // The owner of a byte knows where its columns go, but writing them from there would scatter every store over
    // 64 cache lines.  So the columns are listed in LDS, SG_EMIT at a time, and then every lane writes the entry
    // at its own place in the list: coalesced stores.
    if (total <= SG_EMIT) {         // the usual case: the whole block fits the list
        int at = first_a;
        for (uint32_t w = bits_a; w; w &= w - 1, ++at)
            emit_col[at] = (emit_t)(jbase + __ffs(w) - 1);
        at = first_b;
        for (uint32_t w = bits_b; w; w &= w - 1, ++at)
            emit_col[at] = (emit_t)(SG_CB / 2 + jbase + __ffs(w) - 1);
        lds_barrier();
        for (int q = threadIdx.x; q < total; q += SG_T) {
            const int j = emit_col[q];
            store_streaming(&Ccrd[off + q], col0 + j);
            store_streaming(&Cval[off + q], take(j));
        }
        lds_barrier();
    } else {
        for (int c0 = 0; c0 < total; c0 += SG_EMIT) {
            int at = first_a - c0;
            for (uint32_t w = bits_a; w; w &= w - 1, ++at)
                if (at >= 0 && at < SG_EMIT)
                    emit_col[at] = (emit_t)(jbase + __ffs(w) - 1);
            at = first_b - c0;
            for (uint32_t w = bits_b; w; w &= w - 1, ++at)
                if (at >= 0 && at < SG_EMIT)
                    emit_col[at] = (emit_t)(SG_CB / 2 + jbase + __ffs(w) - 1);
            lds_barrier();
            const int n = total - c0 < SG_EMIT ? total - c0 : SG_EMIT;
            for (int q = threadIdx.x; q < n; q += SG_T) {
                const int j = emit_col[q];
                store_streaming(&Ccrd[off + c0 + q], col0 + j);
                store_streaming(&Cval[off + c0 + q], take(j));
            }
            lds_barrier();
        }
    }
    return total;
}

// MASKED (C<M> = A*B, for the rows whose mask row is too long for the slab kernel's hash table): every product is
// added as without a mask - the LDS adds are not what this kernel waits for - and the mask row decides what leaves:
// before a block's products are walked, the mask row's entries inside the block are set in a bitmap of their own
// (the row is sorted, so they start where the block before ended), and when the block is written out the columns
// outside it are dropped and their accumulators cleared.
// COL: B's columns as 32-bit numbers, or as 16-bit numbers inside their block (see turn_of_slice).
template <bool SEMI, bool MASKED, typename COL>
__global__ __launch_bounds__(SG_T) void spgemm_numeric_dense_kernel(
    int64_t row_begin, int64_t row_end, const int64_t *__restrict__ Apos, const int32_t *__restrict__ Acrd,
    const double *__restrict__ Aval, const COL *__restrict__ Bcrd, const double *__restrict__ Bval,
    const int64_t *__restrict__ Mpos, const int32_t *__restrict__ Mcrd,
    const int64_t *__restrict__ blkptr, int nblk,
    unsigned long long *ticket, RowList list,
    const int64_t *__restrict__ Cpos, int32_t *__restrict__ Ccrd, double *__restrict__ Cval, int reduce_op,
    int mult_op)
{
    __shared__ int64_t row_slot;
    __shared__ int wave_tot[SG_WAVES];
    __shared__ int block_touched[3];            // see visit_flag
    __shared__ unsigned long long mask_next[2]; // where the mask row's entries of a block begin; blocks take turns
    double *acc = reinterpret_cast<double *>(sg_dyn_lds);
    uint32_t *bm = sg_dyn_lds + SG_CB * 2;
    emit_t *emit_col = reinterpret_cast<emit_t *>(bm + SG_CB / 32);
    uint32_t *mbits = reinterpret_cast<uint32_t *>(emit_col + SG_EMIT);
    if constexpr (MASKED) {
        for (int w = threadIdx.x; w < 2 * (SG_CB / 32); w += SG_T)
            mbits[w] = 0;
    }
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    for (int j = threadIdx.x; j < SG_CB; j += SG_T)
        acc[j] = 0.0;
    if (threadIdx.x < SG_CB / 32)
        bm[threadIdx.x] = 0;
    if (threadIdx.x < 3)
        block_touched[threadIdx.x] = 0;
    lds_barrier();
    int visit = 0;
    const int64_t out0 = Cpos[row_begin];
    int64_t t_first, t_end;
    list_range(list, 3, &t_first, &t_end);     // the other heavy rows go to spgemm_numeric_span_kernel
    int64_t t = draw_row<true>(ticket, t_first, &row_slot);
    while (t < t_end) {
        const int64_t i = row_begin + list.rows[t];
        const int64_t as = Apos[i], ae = Apos[i + 1];
        int64_t me = 0;
        if constexpr (MASKED) {
            me = Mpos[i + 1];
            if (threadIdx.x == 0)
                mask_next[0] = mask_next[1] = (unsigned long long)Mpos[i];
            lds_barrier();
        }
        if (as != ae) {
            int64_t off = Cpos[i] - out0;
            // A row of at most one entry of A per lane (nearly all rows) keeps its entries in registers over
            // the blocks: the end of a slice in one block is its start in the next, so a block costs one
            // pointer load per lane, and that load is issued a block ahead.
            const int held = __builtin_amdgcn_readfirstlane((int)(ae - as <= SG_T));
            int64_t h_lo = 0, h_hi = 0;
            double h_a = 0.0;
            int h_pa = 0;
            const int64_t *h_bp = nullptr;
            if (held) {
                const int64_t p = as + wave + (int64_t)lane * SG_WAVES;
                if (p < ae) {
                    h_bp = blkptr + (int64_t)Acrd[p] * (nblk + 1);
                    h_lo = h_bp[0];
                    h_hi = h_bp[1];
                    h_a = Aval[p];
                    h_pa = (int)(p - as + 1);
                }
            }
            for (int cb = 0; cb < nblk; ++cb) {
                const int col0 = cb << SG_CB_LOG;
                uint32_t *mb = mbits + (cb & 1) * (SG_CB / 32);
                if constexpr (MASKED) {
                    // The mask row's entries inside this block: they begin at mask_next[cb & 1], and where they end
                    // goes to the other slot, for the next block (a slot is read in one block and written in the
                    // next one, with the block's barrier in between; it only ever grows along a row).
                    const int64_t lo = (int64_t)mask_next[cb & 1];
                    const int col_end = col0 + SG_CB;
                    if (threadIdx.x == 0)
                        atomicMax(&mask_next[(cb + 1) & 1], (unsigned long long)lo);
                    for (int64_t e = lo + threadIdx.x; e < me; e += SG_T) {
                        const int j = Mcrd[e];
                        if (j >= col_end)
                            break;
                        atomicOr(&mb[(j - col0) >> 5], 1u << ((j - col0) & 31));
                        if (e + 1 == me || Mcrd[e + 1] >= col_end)
                            atomicMax(&mask_next[(cb + 1) & 1], (unsigned long long)(e + 1));
                    }
                }
                int touched = 0;     // did this wavefront add anything to the block
                const auto add = [&](int j, double a, double b, int pa, int64_t q) {
                    dense_add<SEMI, COL>(acc, bm, col0, j, a, b, pa, q, reduce_op, mult_op);
                };
                const auto add4 = [&](auto j, double a, auto v0, auto v1, int pa, int64_t q) {
                    dense_add4<SEMI, COL>(acc, bm, col0, j, a, v0, v1, pa, q, reduce_op, mult_op);
                };
                const auto take = [&](int j) { return dense_take<SEMI>(acc, j, reduce_op, mult_op, as, Aval, Bval); };
                if (held) {
                    int64_t next = h_hi;
                    if (h_bp && cb + 1 < nblk)
                        next = h_bp[cb + 2];
                    touched = for_each_in_slices<true>(h_lo, h_hi, h_a, h_pa, lane, Bcrd, Bval, add, add4);
                    h_lo = h_hi;
                    h_hi = next;
                }
                for (int64_t base = as + wave; !held && base < ae; base += (int64_t)SG_WAVES * 64) {
                    const int64_t left = (ae - base + SG_WAVES - 1) / SG_WAVES;
                    const int cnt = (int)(left < 64 ? left : 64);
                    int64_t lo = 0, hi = 0;
                    double a = 0.0;
                    int pa = 0;
                    if (lane < cnt) {
                        const int64_t p = base + (int64_t)lane * SG_WAVES;
                        const int64_t *bp = blkptr + (int64_t)Acrd[p] * (nblk + 1) + cb;
                        lo = bp[0];
                        hi = bp[1];
                        a = Aval[p];
                        pa = (int)(p - as + 1);
                    }
                    touched |= for_each_in_slices<true>(lo, hi, a, pa, lane, Bcrd, Bval, add, add4);
                }
                const int any = visit_flag(block_touched, visit, touched, lane);
                visit = visit == 2 ? 0 : visit + 1;
                if (any) {
                    off += dense_emit_block<MASKED>(bm, mb, acc, emit_col, wave_tot, lane, wave, col0, Ccrd, Cval,
                                                    take, [&](int) { return off; });
                } else if constexpr (MASKED) {   // the block received no product
                    if (threadIdx.x < SG_CB / 32)        // (the next block's bits go to the other half; the one after
                        mb[threadIdx.x] = 0;             // that comes after the next block's barrier)
                }
            }
        }
        t = draw_row<true>(ticket, t_first, &row_slot);
    }
}

// ---------------------------------------------------------------------------
// The same rows, block by block: the kernel above takes a row through its column blocks, so at any time the
// workgroups of an XCD read the slices of every block and the long rows of B, which most products come from,
// never stay in its L2 (a few hundred rows of an R-MAT graph make over half of the products, but they hold
// tens of megabytes).  Here the tickets go over (column block, row) with the block outermost: all workgroups
// are in the same block at the same time and what they share is that block's slices of the long rows only.
// A row's entries inside a block then leave before the blocks ahead of it are counted, so where they go is
// handed from block to block: before[r * nblk + cb] = the row's entries ahead of block cb, written by the
// workgroup that counted block cb - 1 and awaited by the one that writes block cb.  That one holds a later
// ticket, and a workgroup only ever waits for earlier tickets, which running workgroups hold: the one with the
// earliest unfinished ticket waits for nobody.  The wait is bounded all the same (`patience` polls, after
// which *gave_up is set and the row is wrong: the host then fails the call).
// A ticket is DB_ROWS consecutive rows of the list, so that the loads which lead to a row's slices (its entries
// of A, their block pointers) are issued while the row before is walked.
// ---------------------------------------------------------------------------
struct DenseRow {
    int64_t as;         // first entry of the row of A
    int64_t coff;       // first entry of the row of C, counted from the row block's
    int32_t cnt;        // entries of the row of A
    int32_t pad;
};
constexpr int DB_ROWS = 8;
constexpr int DB_PATIENCE = 1 << 24;

// rows[r] for the nd first rows of the list and before[] in its initial state: nothing ahead of block 0, the rest open
__global__ void spgemm_dense_rows(int64_t row_begin, RowList list, int64_t nd, int nblk, const int64_t *__restrict__ Apos,
                                  const int64_t *__restrict__ Cpos, DenseRow *__restrict__ rows,
                                  int32_t *__restrict__ before)
{
    const int64_t x = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (x < nd * nblk)
        before[x] = x % nblk == 0 ? 0 : -1;
    if (x < nd) {
        const int64_t i = row_begin + list.rows[x];
        DenseRow r;
        r.as = Apos[i];
        r.cnt = (int32_t)(Apos[i + 1] - r.as);         // (the host sends matrices of under 2^30 entries here)
        r.coff = Cpos[i] - Cpos[row_begin];
        r.pad = 0;
        rows[x] = r;
    }
}

template <bool SEMI, typename COL>
__global__ __launch_bounds__(SG_T) void spgemm_numeric_dense_blocks_kernel(
    const DenseRow *__restrict__ rows, int64_t nd, const int32_t *__restrict__ Acrd, const double *__restrict__ Aval,
    const COL *__restrict__ Bcrd, const double *__restrict__ Bval, const int64_t *__restrict__ blkptr, int nblk,
    unsigned long long *ticket, int32_t *before, int patience, int *gave_up, int32_t *__restrict__ Ccrd,
    double *__restrict__ Cval, int reduce_op, int mult_op)
{
    __shared__ int64_t row_slot;
    __shared__ int wave_tot[SG_WAVES];
    __shared__ int block_touched[3];            // see visit_flag
    __shared__ int ahead_slot;                  // the row's entries ahead of the block
    double *acc = reinterpret_cast<double *>(sg_dyn_lds);
    uint32_t *bm = sg_dyn_lds + SG_CB * 2;
    emit_t *emit_col = reinterpret_cast<emit_t *>(bm + SG_CB / 32);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    for (int j = threadIdx.x; j < SG_CB; j += SG_T)
        acc[j] = 0.0;
    if (threadIdx.x < SG_CB / 32)
        bm[threadIdx.x] = 0;
    if (threadIdx.x < 3)
        block_touched[threadIdx.x] = 0;
    lds_barrier();
    int visit = 0;
    const int64_t nchunks = (nd + DB_ROWS - 1) / DB_ROWS;
    const int64_t u_end = nchunks * nblk;
    int64_t u = draw_row<true>(ticket, 0, &row_slot);
    while (u < u_end) {
        const int cb = (int)(u / nchunks);
        const int64_t r0 = (u - cb * nchunks) * DB_ROWS;
        const int nr = (int)(nd - r0 < DB_ROWS ? nd - r0 : DB_ROWS);
        const int col0 = cb << SG_CB_LOG;
        DenseRow mine;
        mine.as = mine.coff = 0;
        mine.cnt = 0;
        if (lane < nr)
            mine = rows[r0 + lane];
        // the entry of A a lane holds of row x of the ticket (of its first SG_T entries: a longer row loads the others
        // as it goes), and the slice of its row of B inside the block
        const auto load_entry = [&](int x, int &k, double &a) {
            k = -1;
            a = 0.0;
            if (x < nr) {
                const int cnt = __builtin_amdgcn_readlane(mine.cnt, x);
                const int p = wave + lane * SG_WAVES;
                if (p < cnt) {
                    const int64_t as = ((int64_t)__builtin_amdgcn_readlane((int)(mine.as >> 32), x) << 32) |
                                       (uint32_t)__builtin_amdgcn_readlane((int)mine.as, x);
                    k = Acrd[as + p];
                    a = Aval[as + p];
                }
            }
        };
        const auto load_slice = [&](int k, int64_t &lo, int64_t &hi) {
            lo = hi = 0;
            if (k >= 0) {
                const int64_t *bp = blkptr + (int64_t)k * (nblk + 1) + cb;
                lo = bp[0];
                hi = bp[1];
            }
        };
        int k0, k1, k2;
        double a0, a1, a2;
        int64_t lo0, hi0, lo1, hi1;
        load_entry(0, k0, a0);
        load_entry(1, k1, a1);
        load_slice(k0, lo0, hi0);
        for (int x = 0; x < nr; ++x) {
            load_slice(k1, lo1, hi1);
            load_entry(x + 2, k2, a2);
            const int cnt = __builtin_amdgcn_readlane(mine.cnt, x);
            const int64_t as = ((int64_t)__builtin_amdgcn_readlane((int)(mine.as >> 32), x) << 32) |
                               (uint32_t)__builtin_amdgcn_readlane((int)mine.as, x);
            const int64_t coff = ((int64_t)__builtin_amdgcn_readlane((int)(mine.coff >> 32), x) << 32) |
                                 (uint32_t)__builtin_amdgcn_readlane((int)mine.coff, x);
            const auto add = [&](int j, double a, double b, int pa, int64_t q) {
                dense_add<SEMI, COL>(acc, bm, col0, j, a, b, pa, q, reduce_op, mult_op);
            };
            const auto add4 = [&](auto j, double a, auto v0, auto v1, int pa, int64_t q) {
                dense_add4<SEMI, COL>(acc, bm, col0, j, a, v0, v1, pa, q, reduce_op, mult_op);
            };
            const auto take = [&](int j) { return dense_take<SEMI>(acc, j, reduce_op, mult_op, as, Aval, Bval); };
            // What lies ahead of this block comes from whoever counted the block before it.  That was many tickets
            // ago as a rule, so the answer is asked for before the walk and the trip to memory it takes is over by
            // the time the walk is; only if it was not there yet is it waited for, behind the walk.
            int32_t *mark = before + (r0 + x) * nblk + cb;
            int early = 0;
            if (threadIdx.x == 0 && cb > 0)
                early = __hip_atomic_fetch_max(mark, -1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const int mine_p = wave + lane * SG_WAVES;          // the entry this lane holds of a batch of SG_T
            int touched = for_each_in_slices<true>(lo0, hi0, a0, mine_p + 1, lane, Bcrd, Bval, add, add4);
            if (cnt > SG_T) {
                // the entries of A beyond the first SG_T, SG_T at a time: a batch's entries are loaded two batches
                // ahead and its slices one, so that a walk does not begin with two trips to memory
                const auto load_more = [&](int base, int &k, double &a) {
                    k = -1;
                    a = 0.0;
                    if (base + mine_p < cnt) {
                        k = Acrd[as + base + mine_p];
                        a = Aval[as + base + mine_p];
                    }
                };
                int kb, kn;
                double ab, an;
                int64_t lob, hib;
                load_more(SG_T, kb, ab);
                load_more(2 * SG_T, kn, an);
                load_slice(kb, lob, hib);
                for (int base = SG_T; base < cnt; base += SG_T) {
                    int64_t lon, hin;
                    load_slice(kn, lon, hin);
                    int kf;
                    double af;
                    load_more(base + 2 * SG_T, kf, af);
                    touched |= for_each_in_slices<true>(lob, hib, ab, base + mine_p + 1, lane, Bcrd, Bval, add, add4);
                    lob = lon;
                    hib = hin;
                    ab = an;
                    kn = kf;
                    an = af;
                }
            }
            const int any = visit_flag(block_touched, visit, touched, lane);
            visit = visit == 2 ? 0 : visit + 1;
            const auto await = [&]() {
                int ahead = early;
                for (int polls = 1; ahead < 0 && polls < patience; ++polls) {
                    __builtin_amdgcn_s_sleep(4);
                    ahead = __hip_atomic_fetch_max(mark, -1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                if (ahead < 0) {
                    __hip_atomic_store(gave_up, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    ahead = 0;
                }
                return ahead;
            };
            const auto hand_on = [&](int ahead) {
                if (cb + 1 < nblk)
                    __hip_atomic_exchange(mark + 1, ahead, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            };
            if (any) {
                if (threadIdx.x == 0)
                    ahead_slot = await();          // (read behind the first barrier of the write-out)
                dense_emit_block<false>(bm, nullptr, acc, emit_col, wave_tot, lane, wave, col0, Ccrd, Cval, take,
                                        [&](int total) {
                                            const int ahead = ahead_slot;
                                            if (threadIdx.x == 0)
                                                hand_on(ahead + total);
                                            return coff + ahead;
                                        });
            } else if (threadIdx.x == 0) {
                hand_on(await());
            }
            k0 = k1;
            a0 = a1;
            lo0 = lo1;
            hi0 = hi1;
            k1 = k2;
            a1 = a2;
        }
        u = draw_row<true>(ticket, 0, &row_slot);
    }
}

// ---------------------------------------------------------------------------
// Heavy rows that are not wide: a row with 10^4..10^5 products is the union of a few long rows of B with hardly
// a column in common, so each of its 64 column blocks receives a few hundred products and a block visit of the
// kernel above costs more in barriers and write-out than in products.  Here a visit spans up to SP_BLOCKS column
// blocks and keeps the values compact: a first pass over the products sets the span's bitmap in LDS, a prefix
// sum over the bitmap gives every column its rank, and a second pass adds each product at the rank of its column
// (two LDS reads and one fp64 LDS atomic).  The values then leave in rank order, which is column order, and the
// columns come from the bitmap.  The compact array holds SP_CAP = 16384 entries; a span that holds more is cut
// at the last block boundary that fits (one block always does), so the kernel is right for any row and merely
// slow for wide ones.
// ---------------------------------------------------------------------------
constexpr int SP_BLOCKS = 8;                              // column blocks per visit at most
constexpr int SP_BLOCK_WORDS = SG_CB / 32;                // bitmap words of one block
constexpr int SP_WORDS = SP_BLOCKS * SP_BLOCK_WORDS;      // bitmap words of a span
constexpr int SP_WPT = SP_WORDS / SG_T;                   // consecutive bitmap words per thread
constexpr int SP_CAP = SG_CB;                             // entries of C per visit at most
constexpr int SP_CHUNK = 64 * SG_LONG_LOADS;              // entries of a slice that a wavefront takes in one turn
constexpr size_t SG_SPAN_LDS = (size_t)SP_CAP * 8 + (size_t)SP_WORDS * 4 + (size_t)SP_WORDS * 2;   // values, bitmap, ranks
static_assert(((size_t)SP_CAP * 8) % 8 == 0 && ((size_t)SP_WORDS * 4) % 4 == 0,
              "the span kernel's values (fp64) come first in its LDS, bitmap and ranks follow on word boundaries");
static_assert(SP_WORDS % SG_T == 0 && SP_BLOCK_WORDS % SP_WPT == 0 && SP_CAP >= SG_CB && SP_CAP <= 65535,
              "a thread's words lie in one block, one block fits the value array, ranks fit 16 bits");

template <bool SEMI>
__global__ __launch_bounds__(SG_T) void spgemm_numeric_span_kernel(
    int64_t row_begin, int64_t row_end, const int64_t *__restrict__ Apos, const int32_t *__restrict__ Acrd,
    const double *__restrict__ Aval, const int32_t *__restrict__ Bcrd, const double *__restrict__ Bval,
    const int64_t *__restrict__ blkptr, int nblk,
    unsigned long long *ticket, RowList list,
    const int64_t *__restrict__ Cpos, int32_t *__restrict__ Ccrd, double *__restrict__ Cval, int reduce_op,
    int mult_op)
{
    __shared__ int64_t row_slot;
    __shared__ int wave_tot[SG_WAVES];
    __shared__ int blk_pre[SP_BLOCKS + 1];      // entries of the span before each of its blocks, and in all
    __shared__ int span_touched[3];             // see visit_flag below
    double *val = reinterpret_cast<double *>(sg_dyn_lds);
    uint32_t *bm = sg_dyn_lds + SP_CAP * 2;
    uint16_t *pre = reinterpret_cast<uint16_t *>(bm + SP_WORDS);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    for (int j = threadIdx.x; j < SP_CAP; j += SG_T)
        val[j] = 0.0;
    for (int w = threadIdx.x; w < SP_WORDS; w += SG_T)
        bm[w] = 0;
    if (threadIdx.x < 3)
        span_touched[threadIdx.x] = 0;
    lds_barrier();
    int visit = 0;
    const int64_t out0 = Cpos[row_begin];
    int64_t t_first, t_end;
    list_range(list, 4, &t_first, &t_end);
    int64_t t = draw_row<true>(ticket, t_first, &row_slot);
    while (t < t_end) {
        const int64_t i = row_begin + list.rows[t];
        const int64_t as = Apos[i], ae = Apos[i + 1];
        if (ae - as == 1) {
            // one entry of A: the row of C is that row of B times the entry (0 + a * b, as an accumulator that
            // starts at zero gives it).  70,000 rows of the R-MAT product at scale 20 are like that, each the
            // copy of a hub's row.
            const int64_t *bp = blkptr + (int64_t)Acrd[as] * (nblk + 1);
            const int64_t bs = bp[0], len = bp[nblk] - bs, off = Cpos[i] - out0;
            const double a = Aval[as];
            for (int64_t q = threadIdx.x; q < len; q += SG_T) {
                store_streaming(&Ccrd[off + q], Bcrd[bs + q]);
                if constexpr (SEMI) {        // what the reference's accumulator holds after this one product
                    const double e = semiring_mult(mult_op, a, Bval[bs + q]);
                    store_streaming(&Cval[off + q], reduce_op == SR_PLUS  ? 0.0 + e
                                                    : reduce_op == SR_MAX ? (f64_key(e) < f64_key(0.0) ? 0.0 : e)
                                                                          : e);
                } else {
                    store_streaming(&Cval[off + q], 0.0 + a * Bval[bs + q]);
                }
            }
        } else if (as != ae) {
            int64_t off = Cpos[i] - out0;
            // A row of at most one entry of A per lane (nearly all rows) keeps the entry, the place of its block
            // pointers and the slice of the span in registers; the end of the next span is loaded a visit ahead.
            // A row of at most 64 entries of A (the usual heavy row that is not wide has 5..140) is held whole by
            // every wavefront, entry l in lane l, and its slices are dealt to the wavefronts in chunks of
            // SP_CHUNK entries: with an entry per wavefront, 5 entries would leave 11 wavefronts idle.
            const int held = __builtin_amdgcn_readfirstlane((int)(ae - as <= SG_T));
            const int small = __builtin_amdgcn_readfirstlane((int)(ae - as <= 64));
            double h_a = 0.0;
            int h_pa = 0;
            const int64_t *h_bp = nullptr;
            int64_t h_lo = 0, h_hi = 0;
            if (held) {
                const int64_t p = small ? as + lane : as + wave + (int64_t)lane * SG_WAVES;
                if (p < ae) {
                    h_bp = blkptr + (int64_t)Acrd[p] * (nblk + 1);
                    h_a = Aval[p];
                    h_pa = (int)(p - as + 1);
                    h_lo = h_bp[0];
                    h_hi = h_bp[nblk < SP_BLOCKS ? nblk : SP_BLOCKS];
                }
            }
            // f over the products of the row whose columns lie in the blocks [cbf, cbt); a held row's slice of these
            // blocks is [held_lo, held_hi)
            const auto walk = [&](int cbf, int cbt, int64_t held_lo, int64_t held_hi, auto values, auto f, auto f4) -> int {
                constexpr bool VALUES = decltype(values)::value;
                int touched = 0;
                if (small) {
                    const int mine = (int)((held_hi - held_lo + SP_CHUNK - 1) / SP_CHUNK);
                    const int upto = wave_inclusive_scan(mine);             // chunks of the entries 0..lane
                    const int chunks = __builtin_amdgcn_readlane(upto, 63);
                    touched = chunks > 0;
                    for (int g = wave; g < chunks; g += SG_WAVES) {
                        const int e = __builtin_ctzll(__ballot(upto > g));   // the entry that chunk g belongs to
                        const int c = g - (__builtin_amdgcn_readlane(upto, e) - __builtin_amdgcn_readlane(mine, e));
                        const int64_t s = readlane_i64(held_lo, e) + (int64_t)c * SP_CHUNK;
                        const int64_t left = readlane_i64(held_hi, e) - s;
                        if (left >= SP_CHUNK)
                            full_turn_of_slice<VALUES>(s, lane, readlane_d(h_a, e), __builtin_amdgcn_readlane(h_pa, e), Bcrd,
                                                       Bval, f4);
                        else
                            turn_of_slice<VALUES>(s, lane, left, readlane_d(h_a, e), __builtin_amdgcn_readlane(h_pa, e),
                                                  Bcrd, Bval, f);
                    }
                } else if (held)
                    touched = for_each_in_slices<VALUES>(held_lo, held_hi, h_a, h_pa, lane, Bcrd, Bval, f, f4);
                for (int64_t base = as + wave; !held && base < ae; base += (int64_t)SG_WAVES * 64) {
                    const int64_t left = (ae - base + SG_WAVES - 1) / SG_WAVES;
                    const int cnt = (int)(left < 64 ? left : 64);
                    int64_t lo = 0, hi = 0;
                    double a = 0.0;
                    int pa = 0;
                    if (lane < cnt) {
                        const int64_t p = base + (int64_t)lane * SG_WAVES;
                        const int64_t *bp = blkptr + (int64_t)Acrd[p] * (nblk + 1);
                        lo = bp[cbf];
                        hi = bp[cbt];
                        a = Aval[p];
                        pa = (int)(p - as + 1);
                    }
                    touched |= for_each_in_slices<VALUES>(lo, hi, a, pa, lane, Bcrd, Bval, f, f4);
                }
                return touched;
            };
            int cb = 0;
            while (cb < nblk) {
                const int nbv = nblk - cb < SP_BLOCKS ? nblk - cb : SP_BLOCKS;
                const int col0 = cb << SG_CB_LOG;
                int64_t h_next = h_hi;      // where the span after this one ends
                if (h_bp && cb + nbv < nblk)
                    h_next = h_bp[cb + nbv + SP_BLOCKS < nblk ? cb + nbv + SP_BLOCKS : nblk];
                const int touched = walk(cb, cb + nbv, h_lo, h_hi, std::false_type{},
                                         [&](int j, double, double, int, int64_t) {
                    j -= col0;
                    atomicOr(&bm[j >> 5], 1u << (j & 31));
                }, [&](sg_i4u j4, double, sg_d2u, sg_d2u, int, int64_t) {
                    // four consecutive entries of a sorted row: the bits that fall into one word go there together
                    const int j[4] = {j4.x - col0, j4.y - col0, j4.z - col0, j4.w - col0};
                    int w = j[0] >> 5;
                    uint32_t bits = 1u << (j[0] & 31);
#pragma unroll
                    for (int x = 1; x < 4; ++x) {
                        if ((j[x] >> 5) != w) {
                            atomicOr(&bm[w], bits);
                            w = j[x] >> 5;
                            bits = 0u;
                        }
                        bits |= 1u << (j[x] & 31);
                    }
                    atomicOr(&bm[w], bits);
                });
                const int any = visit_flag(span_touched, visit, touched, lane);
                visit = visit == 2 ? 0 : visit + 1;
                int nb = nbv;
                if (any) {
                    // ranks: thread t owns the words [SP_WPT * t, SP_WPT * (t + 1))
                    uint32_t w[SP_WPT];
                    int mine = 0;
#pragma unroll
                    for (int k = 0; k < SP_WPT; ++k) {
                        w[k] = bm[threadIdx.x * SP_WPT + k];
                        mine += __popc(w[k]);
                    }
                    const int inc = wave_inclusive_scan(mine);
                    if (lane == 63)
                        wave_tot[wave] = inc;
                    lds_barrier();
                    const int tots = wave_inclusive_scan(lane < SG_WAVES ? wave_tot[lane] : 0);
                    const int all = __builtin_amdgcn_readlane(tots, SG_WAVES - 1);
                    const int before = (wave ? __builtin_amdgcn_readlane(tots, wave - 1) : 0) + inc - mine;
                    int run = before;
#pragma unroll
                    for (int k = 0; k < SP_WPT; ++k) {
                        pre[threadIdx.x * SP_WPT + k] = (uint16_t)(run < 65535 ? run : 65535);    // exact below the cut
                        run += __popc(w[k]);
                    }
                    if (threadIdx.x % (SP_BLOCK_WORDS / SP_WPT) == 0)
                        blk_pre[threadIdx.x / (SP_BLOCK_WORDS / SP_WPT)] = before;
                    if (threadIdx.x == SG_T - 1)
                        blk_pre[SP_BLOCKS] = all;
                    lds_barrier();
                    // the cut: as many blocks as fit the value array (blocks the span does not have are empty)
                    nb = 1;
                    for (int b = 2; b <= nbv; ++b)
                        nb = __builtin_amdgcn_readfirstlane(blk_pre[b]) <= SP_CAP ? b : nb;
                    const int total = __builtin_amdgcn_readfirstlane(blk_pre[nb]);
                    if (nb < nbv) {              // cut: this visit ends, and the next span starts, at block cb + nb
                        if (h_bp) {
                            h_hi = h_bp[cb + nb];
                            h_next = h_bp[cb + nb + SP_BLOCKS < nblk ? cb + nb + SP_BLOCKS : nblk];
                        }
                    }
                    const auto add_at_rank = [&](int j, double a, double b, int pa, int64_t q) {
                        j -= col0;
                        const uint32_t below = bm[j >> 5] & ((1u << (j & 31)) - 1u);
                        const int r = pre[j >> 5] + __popc(below);
                        if constexpr (SEMI)
                            semiring_lds_add(&val[r], reduce_op, mult_op, a, b, pa, q);
                        else
                            __hip_atomic_fetch_add(&val[r], a * b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    };
                    walk(cb, cb + nb, h_lo, h_hi, std::true_type{}, add_at_rank,
                         [&](sg_i4u j4, double a, sg_d2u v0, sg_d2u v1, int pa, int64_t q) {
                        add_at_rank(j4.x, a, v0.x, pa, q);
                        add_at_rank(j4.y, a, v0.y, pa, q + 1);
                        add_at_rank(j4.z, a, v1.x, pa, q + 2);
                        add_at_rank(j4.w, a, v1.y, pa, q + 3);
                    });
                    lds_barrier();
                    for (int q = threadIdx.x; q < total; q += SG_T) {
                        if constexpr (SEMI)
                            store_streaming(&Cval[off + q],
                                            semiring_lds_value(reinterpret_cast<unsigned long long *>(val)[q], reduce_op,
                                                               mult_op, as, Aval, Bval));
                        else
                            store_streaming(&Cval[off + q], val[q]);
                    }
                    lds_barrier();
                    // the values are out: their array now takes the list of the columns, so that these leave
                    // through coalesced stores too (from their owners they would scatter, four bytes per lane)
                    uint32_t *cols = reinterpret_cast<uint32_t *>(val);
                    int at = before;
#pragma unroll
                    for (int k = 0; k < SP_WPT; ++k) {
                        const int wi = threadIdx.x * SP_WPT + k;
                        if (wi < nb * SP_BLOCK_WORDS)
                            for (uint32_t bits = w[k]; bits; bits &= bits - 1)
                                cols[at++] = (uint32_t)(wi * 32 + __ffs(bits) - 1);
                        bm[wi] = 0;             // also the words beyond the cut: the next visit sets them again
                    }
                    lds_barrier();
                    for (int q = threadIdx.x; q < total; q += SG_T)
                        store_streaming(&Ccrd[off + q], col0 + (int)cols[q]);
                    lds_barrier();
                    for (int q = threadIdx.x; q < total; q += SG_T)
                        val[q] = 0.0;           // nobody adds into it before the next visit's three barriers
                    off += total;
                }
                cb += nb;
                h_lo = h_hi;
                h_hi = h_next;
            }
        }
        t = draw_row<true>(ticket, t_first, &row_slot);
    }
}

// ---------------------------------------------------------------------------
// Masked SpGEMM + SUM without the output: rowsum[i] = sum over products of row
// i that fall on a stored entry of mask row i.  Per-lane partial sums are
// combined in a fixed order, so the result does not depend on scheduling.
// ---------------------------------------------------------------------------
template <bool BM_LDS>
__global__ __launch_bounds__(SG_T) void spgemm_masked_sum_kernel(
    int64_t nrows, const int64_t *__restrict__ Apos, const int32_t *__restrict__ Acrd,
    const double *__restrict__ Aval, const int64_t *__restrict__ Bpos, const int32_t *__restrict__ Bcrd,
    const double *__restrict__ Bval, const int64_t *__restrict__ Mpos, const int32_t *__restrict__ Mcrd,
    int logW, uint32_t *__restrict__ gbm, unsigned long long *ticket, RowList list, double *__restrict__ rowsum)
{
    // takes the rows with work from the heavy end of the list; spgemm_masked_sum_small_kernel comes from the other
    __shared__ int64_t row_slot;
    __shared__ double wave_part[SG_WAVES];
    uint32_t *bm;
    if constexpr (BM_LDS)
        bm = sg_dyn_lds;
    else
        bm = gbm + (size_t)blockIdx.x * (size_t)(SG_T * ((1 << logW) + 1));
    const BmAddr ad{logW};
    const int nwords = SG_T * ((1 << logW) + 1);
    if constexpr (BM_LDS) {
        for (int w = threadIdx.x; w < nwords; w += SG_T)
            bm[w] = 0;
    }
    __syncthreads();
    int64_t t_first, t_end;
    list_range(list, 2, &t_first, &t_end);
    int64_t tk = draw_front(ticket, t_end, &row_slot);
    while (tk < t_end) {
        const int64_t i = list.rows[tk];      // rows outside the list keep the zero the host put there
        const int64_t as = Apos[i], ae = Apos[i + 1];
        const int64_t ms = Mpos[i], me = Mpos[i + 1];
        const bool work = as != ae && ms != me;
        if (work) {
        for (int64_t t = ms + threadIdx.x; t < me; t += SG_T)
            atomicOr(&bm[ad.word(Mcrd[t])], ad.bit(Mcrd[t]));
        __syncthreads();
        double part = 0.0;
        for_each_product_probed<true>(as, ae, Acrd, Aval, Bpos, Bcrd, [&](int j) {
            if constexpr (BM_LDS)
                return bm[ad.word(j)];
            else
                return atomicOr(&bm[ad.word(j)], 0u);
        }, [&](int j, int64_t q, uint32_t word) {
            MaskHit h{-1, 0.0};
            if (word & ad.bit(j)) {      // the value is fetched for hits only
                h.at = 0;
                h.b = Bval[q];
            }
            return h;
        }, [&](int, int64_t, double a, int64_t, int64_t, MaskHit h) {
            if (h.at >= 0)
                part += a * h.b;
        });
        part = wave_sum_f64(part);
        if ((threadIdx.x & 63) == 0)
            wave_part[threadIdx.x >> 6] = part;
        __syncthreads();
        if (threadIdx.x == 0) {
            double total = 0.0;
            for (int w = 0; w < SG_WAVES; ++w)
                total += wave_part[w];
            rowsum[i] = total;
        }
        for (int64_t t = ms + threadIdx.x; t < me; t += SG_T)
            atomicAnd(&bm[ad.word(Mcrd[t])], 0u);
        }   // work
        tk = draw_front(ticket, t_end, &row_slot);     // its barriers also close this row's bitmap clean-up
    }
}

// ---------------------------------------------------------------------------
// The same sum for rows with few products: one wavefront per row, no workgroup
// barrier anywhere.  A row of a thousand products spends more time on the
// ticket, bitmap and reduction barriers of the kernel above than on its
// products.  Here the mask row goes into a small hash table in LDS that belongs
// to the wavefront; the neighbours of the row are taken one at a time and the
// lanes walk along that neighbour's row of B, probing the table.  A mask row too
// long for the table is searched by bisection in memory instead.
// ---------------------------------------------------------------------------
constexpr int SM_WAVES = 4;                    // wavefronts per workgroup
constexpr int SM_SLOTS = 256;                  // hash slots per wavefront (1 KB: four such workgroups fit a CU beside
                                               // one workgroup of the kernel above and its 132 KB bitmap)
constexpr int SM_MASK_MAX = 96;                // longest mask row that goes into the table
constexpr int SM_BATCH = 16;                   // rows a wavefront claims at a time in the lighter half of the list

__device__ inline int sm_hash(int j) { return (int)(((uint32_t)j * 2654435761u) >> 24) & (SM_SLOTS - 1); }

__global__ __launch_bounds__(SM_WAVES * 64) void spgemm_masked_sum_small_kernel(
    const int64_t *__restrict__ Apos, const int32_t *__restrict__ Acrd, const double *__restrict__ Aval,
    const int64_t *__restrict__ Bpos, const int32_t *__restrict__ Bcrd, const double *__restrict__ Bval,
    const int64_t *__restrict__ Mpos, const int32_t *__restrict__ Mcrd, unsigned long long *ticket, RowList list,
    double *__restrict__ rowsum)
{
    __shared__ int table[SM_WAVES][SM_SLOTS];
    const int lane = threadIdx.x & 63;
    int *tab = table[threadIdx.x >> 6];
    for (int s = lane; s < SM_SLOTS; s += 64)
        tab[s] = -1;
    int64_t t_first, t_end;
    list_range(list, 2, &t_first, &t_end);
    int take = SM_BATCH;
    int64_t mine_next = 0, mine_end = 0;     // the rows t_end - 1 - b, b in [mine_next, mine_end), are this wavefront's
    for (;;) {
        if (mine_next == mine_end) {
            // rows from the light end of the list (see draw_front): SM_BATCH at a time in the lighter half of the
            // list - rows of a few thousand products at most, and 600,000 draws on one word are what the L2 does
            // in the time the whole count takes - a quarter of that in the next quarter, then one by one: a
            // batch of rows near the meeting point would keep one wavefront for long
            unsigned long long drawn = 0;
            if (lane == 0)
                drawn = atomicAdd(ticket, (unsigned long long)take << 32);
            const int64_t f = (int64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(drawn & 0xffffffffu));
            const int64_t b = (int64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(drawn >> 32));
            if (f + b >= t_end)
                break;
            mine_next = b;
            mine_end = b + take < t_end - f ? b + take : t_end - f;     // what the front had not reached
            const int64_t taken = b + take;
            take = taken < t_end / 2 ? SM_BATCH : taken < t_end - t_end / 4 ? SM_BATCH / 4 : 1;
        }
        const int64_t tk = t_end - 1 - mine_next;
        ++mine_next;
        const int64_t i = list.rows[tk];
        const int64_t as = Apos[i], ae = Apos[i + 1], ms = Mpos[i], me = Mpos[i + 1];
        if (as == ae || ms == me)
            continue;               // rowsum[i] keeps the zero the host put there
        const bool hashed = me - ms <= SM_MASK_MAX;
        if (hashed)
            for (int64_t t = ms + lane; t < me; t += 64) {
                const int j = Mcrd[t];
                int h = sm_hash(j);
                while (atomicCAS(&tab[h], -1, j) != -1)
                    h = (h + 1) & (SM_SLOTS - 1);
            }
        double part = 0.0;
        for (int64_t p0 = as; p0 < ae; p0 += 64) {
            // up to 64 neighbours at a time: lane l holds neighbour p0 + l, its value and its row of B
            const int cnt = (int)(ae - p0 < 64 ? ae - p0 : 64);
            int64_t bs = 0, be = 0;
            double a = 0.0;
            if (lane < cnt) {
                const int k = Acrd[p0 + lane];
                bs = Bpos[k];
                be = Bpos[k + 1];
                a = Aval[p0 + lane];
            }
            auto probe = [&](int j, int64_t q, double al) {
                bool hit = false;
                if (hashed) {
                    int h = sm_hash(j);
                    for (int v = tab[h]; v != -1; v = tab[h]) {
                        if (v == j) {
                            hit = true;
                            break;
                        }
                        h = (h + 1) & (SM_SLOTS - 1);
                    }
                } else {
                    int64_t lo = ms, hi = me;
                    while (lo < hi) {
                        const int64_t mid = (lo + hi) >> 1;
                        if (Mcrd[mid] < j)
                            lo = mid + 1;
                        else
                            hi = mid;
                    }
                    hit = lo < me && Mcrd[lo] == j;
                }
                if (hit)
                    part += al * Bval[q];
            };
            // rows of B with 64 entries and more take the whole wavefront, one at a time; shorter ones (a row
            // of the lower triangle holds 15 entries on average) go to the four 16-lane quarters, four at a time.
            // (Laying all products of the row end to end, lane x taking product x after a bisection over the
            // running totals, fills every lane and was slower: 11.0 against 10.0 ms - the kernel is bound by
            // instructions per product, not by idle lanes.)
            unsigned long long big = __ballot(be - bs >= 64);
            unsigned long long todo = __ballot(bs < be && be - bs < 64);
            while (big) {
                const int l = __builtin_ctzll(big);
                big &= big - 1;
                const int64_t s = readlane_i64(bs, l), e = readlane_i64(be, l);
                const double al = readlane_d(a, l);
                for (int64_t q = s + lane; q < e; q += 256) {      // all loads of a turn first, then the probes
                    int j[4];
#pragma unroll
                    for (int x = 0; x < 4; ++x)
                        j[x] = q + 64 * x < e ? Bcrd[q + 64 * x] : 0;
#pragma unroll
                    for (int x = 0; x < 4; ++x)
                        if (q + 64 * x < e)
                            probe(j[x], q + 64 * x, al);
                }
            }
            const int quarter = lane >> 4, sub = lane & 15;
            while (todo) {
                int pick = -1;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int l = todo ? __builtin_ctzll(todo) : -1;
                    todo = todo ? (todo & (todo - 1)) : 0;
                    pick = quarter == g ? l : pick;
                }
                const int src = pick < 0 ? lane : pick;
                const int64_t s = ((int64_t)__shfl((int)(bs >> 32), src, 64) << 32) |
                                  (uint32_t)__shfl((int)(bs & 0xffffffff), src, 64);
                const int64_t e = ((int64_t)__shfl((int)(be >> 32), src, 64) << 32) |
                                  (uint32_t)__shfl((int)(be & 0xffffffff), src, 64);
                const double al = __hiloint2double(__shfl(__double2hiint(a), src, 64),
                                                   __shfl(__double2loint(a), src, 64));
                int j[4];                   // a row here has fewer than 64 entries: four per lane cover it
#pragma unroll
                for (int x = 0; x < 4; ++x)
                    j[x] = pick >= 0 && s + sub + 16 * x < e ? Bcrd[s + sub + 16 * x] : 0;
#pragma unroll
                for (int x = 0; x < 4; ++x)
                    if (pick >= 0 && s + sub + 16 * x < e)
                        probe(j[x], s + sub + 16 * x, al);
            }
        }
        part = wave_sum_f64(part);
        if (lane == 0)
            rowsum[i] = part;
        if (hashed)
            for (int s = lane; s < SM_SLOTS; s += 64)
                tab[s] = -1;
    }
}

// ---------------------------------------------------------------------------
// The same sums when every stored value of B is one number b (a pattern matrix): a product that meets the mask
// adds a * b whatever its place in the row of B, so a row of B only has to be counted - how many of its columns
// are in the mask row - and the count times a * b is what it contributes.  No value is fetched, nothing is
// carried from the look-up to a later visit, and the walk shrinks to a load, an LDS read and a bit test per
// product.  (Sums of whole numbers, as in a triangle count, are the same in either form; otherwise the two differ
// by rounding, each within the bound the unmasked forms keep.)
// ---------------------------------------------------------------------------
__device__ __forceinline__ int bitmap_bit(const uint32_t *bm, int j)
{
    return (int)((bm[(uint32_t)j >> 5] >> ((uint32_t)j & 31u)) & 1u);
}
__device__ __forceinline__ int bitmap_bits4(const uint32_t *bm, sg_i4u j)
{
    const uint32_t w0 = bm[(uint32_t)j.x >> 5], w1 = bm[(uint32_t)j.y >> 5], w2 = bm[(uint32_t)j.z >> 5],
                   w3 = bm[(uint32_t)j.w >> 5];
    return (int)(((w0 >> ((uint32_t)j.x & 31u)) & 1u) + ((w1 >> ((uint32_t)j.y & 31u)) & 1u) +
                 ((w2 >> ((uint32_t)j.z & 31u)) & 1u) + ((w3 >> ((uint32_t)j.w & 31u)) & 1u));
}
// What a lane holds of a turn in flight: up to four 16-byte loads (four consecutive columns each) of the row of
// B its group of lanes is on, one more column if the row's length is not a multiple of four, and the value
// a * b every hit of this row is worth.
struct IsoTurn {
    sg_i4u q[4];
    int tail;
    uint32_t ok;        // bit x: q[x] holds columns; bit 4: tail does
    double at;
};
// The loads of a turn.  `row` is the lane's row of B, `first` the first group of four columns the lane takes and
// `stride` the distance to its next one, nq the number of full groups of four in the row; rest = the columns
// beyond them if this is the row's last turn (else 0), taken by the first lanes of the group (sub = the lane's
// number inside it).
__device__ __forceinline__ void iso_issue(IsoTurn &t, const int32_t *__restrict__ row, int first, int stride, int nq,
                                          int rest, int sub, double at)
{
    t.ok = 0;
    t.at = at;
    t.tail = 0;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        const int qi = first + stride * x;
        t.q[x] = sg_i4u{0, 0, 0, 0};
        if (qi < nq) {
            t.q[x] = *reinterpret_cast<const sg_i4u *>(row + 4 * qi);
            t.ok |= 1u << x;
        }
    }
    if (sub < rest) {
        t.tail = row[4 * nq + sub];
        t.ok |= 16u;
    }
}
template <typename PROBE>
__device__ __forceinline__ void iso_consume(const IsoTurn &t, const PROBE &probe, double &part)
{
    int hits = 0;
#pragma unroll
    for (int x = 0; x < 4; ++x)
        if (t.ok & (1u << x))
            hits += probe.four(t.q[x]);
    if (t.ok & 16u)
        hits += probe.one(t.tail);
    if (hits)                   // a row without hits adds nothing, whatever its value (0 * inf would be NaN)
        part += (double)hits * t.at;
}
// `todo` names lanes that hold a row of B each; the next G of them go to the G groups of 64 / G lanes of the
// wavefront.  Returns the lane whose row this lane's group takes, or -1.
template <int G>
__device__ __forceinline__ int iso_pick(unsigned long long &todo, int lane)
{
    int pick = -1;
    const int group = lane / (64 / G);
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int t = todo ? __builtin_ctzll(todo) : -1;
        todo = todo ? (todo & (todo - 1)) : 0;
        pick = group == g ? t : pick;
    }
    return pick;
}

// The walk of one output row by a team of TEAM wavefronts (this is wavefront `wave` of it).  The entries of A's
// row are dealt to the wavefronts one at a time, 64 per wavefront and pass.  What bounds a walk like this is
// not the look-ups but the wait for a row of B to arrive, so rows are taken several at a time and a turn
// ahead: rows of 512 entries and more by the whole wavefront, 1024 columns per turn; rows of 256 and more two at
// a time, one per half; shorter ones four at a time, one per 16-lane quarter; and the loads of a turn are issued
// before the look-ups of the turn before it, across rows.  probe.four(j4) / probe.one(j) say how many of the
// columns are in the mask row.  Returns the lane's share of the sum.
template <int TEAM, typename PROBE>
__device__ __forceinline__ double iso_walk(int64_t as, int64_t ae, const int32_t *__restrict__ Acrd,
                                           const double *__restrict__ Aval, const int64_t *__restrict__ Bpos,
                                           const int32_t *__restrict__ Bcrd, double biso, const PROBE &probe, int wave,
                                           int lane)
{
    double part = 0.0;
    IsoTurn pend;
    pend.ok = 0;
    pend.at = 0.0;
    pend.tail = 0;
#pragma unroll
    for (int x = 0; x < 4; ++x)
        pend.q[x] = sg_i4u{0, 0, 0, 0};
    for (int64_t base = as + wave; base < ae; base += (int64_t)TEAM * 64) {
        const int64_t left = (ae - base + TEAM - 1) / TEAM;     // my entries from here on
        const int cnt = (int)(left < 64 ? left : 64);
        int64_t bs = 0;
        int len = 0;
        double a = 0.0;
        if (lane < cnt) {
            const int64_t p = base + (int64_t)lane * TEAM;
            const int k = Acrd[p];
            bs = Bpos[k];
            len = (int)(Bpos[k + 1] - bs);      // a row holds fewer entries than the matrix has columns: < 2^31
            a = Aval[p] * biso;
        }
        unsigned long long big = __ballot(len >= 512);
        unsigned long long mid = __ballot(len >= 256 && len < 512);
        unsigned long long small = __ballot(len > 0 && len < 256);
        while (big) {
            const int t = __builtin_ctzll(big);
            big &= big - 1;
            const int32_t *row = Bcrd + readlane_i64(bs, t);
            const int n = __builtin_amdgcn_readlane(len, t);
            const double at = readlane_d(a, t);
            const int nq = n >> 2;
            for (int tb = 0; tb == 0 || tb < nq; tb += 256) {
                IsoTurn now;
                iso_issue(now, row, tb + lane, 64, nq, tb + 256 >= nq ? (n & 3) : 0, lane, at);
                iso_consume(pend, probe, part);
                pend = now;
            }
        }
        while (mid) {
            const int pick = iso_pick<2>(mid, lane);
            const int src = pick < 0 ? lane : pick;
            // by every lane: a lane whose group sits this round out may be another's source
            const int64_t s = ((int64_t)__shfl((int)(bs >> 32), src, 64) << 32) |
                              (uint32_t)__shfl((int)(bs & 0xffffffff), src, 64);
            const int n_src = __shfl(len, src, 64);
            const double at = __hiloint2double(__shfl(__double2hiint(a), src, 64), __shfl(__double2loint(a), src, 64));
            const int n = pick < 0 ? 0 : n_src;
            IsoTurn now;
            iso_issue(now, Bcrd + s, lane & 31, 32, n >> 2, n & 3, lane & 31, at);
            iso_consume(pend, probe, part);
            pend = now;
        }
        while (small) {
            const int pick = iso_pick<4>(small, lane);
            const int src = pick < 0 ? lane : pick;
            const int64_t s = ((int64_t)__shfl((int)(bs >> 32), src, 64) << 32) |
                              (uint32_t)__shfl((int)(bs & 0xffffffff), src, 64);
            const int n_src = __shfl(len, src, 64);
            const double at = __hiloint2double(__shfl(__double2hiint(a), src, 64), __shfl(__double2loint(a), src, 64));
            const int n = pick < 0 ? 0 : n_src;
            IsoTurn now;
            iso_issue(now, Bcrd + s, lane & 15, 16, n >> 2, n & 3, lane & 15, at);
            iso_consume(pend, probe, part);
            pend = now;
        }
    }
    iso_consume(pend, probe, part);
    return part;
}

struct BitmapProbe {
    const uint32_t *bm;
    __device__ __forceinline__ int one(int j) const { return bitmap_bit(bm, j); }
    __device__ __forceinline__ int four(sg_i4u j) const { return bitmap_bits4(bm, j); }
};

__global__ __launch_bounds__(SG_T) void spgemm_masked_sum_iso_kernel(
    const int64_t *__restrict__ Apos, const int32_t *__restrict__ Acrd, const double *__restrict__ Aval,
    const int64_t *__restrict__ Bpos, const int32_t *__restrict__ Bcrd, double biso,
    const int64_t *__restrict__ Mpos, const int32_t *__restrict__ Mcrd, int nwords, unsigned long long *ticket,
    RowList list, double *__restrict__ rowsum)
{
    // the workgroup kernel: rows from the heavy end of the list, the mask row as a bitmap of nwords words in LDS
    __shared__ int64_t row_slot;
    __shared__ double wave_part[SG_WAVES];
    uint32_t *bm = sg_dyn_lds;
    for (int w = threadIdx.x; w < nwords; w += SG_T)
        bm[w] = 0;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int64_t t_first, t_end;
    list_range(list, 2, &t_first, &t_end);
    int64_t tk = draw_front(ticket, t_end, &row_slot);
    while (tk < t_end) {
        const int64_t i = list.rows[tk];      // rows outside the list keep the zero the host put there
        const int64_t as = Apos[i], ae = Apos[i + 1];
        const int64_t ms = Mpos[i], me = Mpos[i + 1];
        const bool work = as != ae && ms != me;
        if (work) {
            for (int64_t t = ms + threadIdx.x; t < me; t += SG_T) {
                const uint32_t j = (uint32_t)Mcrd[t];
                atomicOr(&bm[j >> 5], 1u << (j & 31u));
            }
            __syncthreads();
            double part = iso_walk<SG_WAVES>(as, ae, Acrd, Aval, Bpos, Bcrd, biso, BitmapProbe{bm}, wave, lane);
            part = wave_sum_f64(part);
            if (lane == 0)
                wave_part[wave] = part;
            __syncthreads();
            if (threadIdx.x == 0) {
                double total = 0.0;
                for (int w = 0; w < SG_WAVES; ++w)
                    total += wave_part[w];
                rowsum[i] = total;
            }
            for (int64_t t = ms + threadIdx.x; t < me; t += SG_T)
                bm[(uint32_t)Mcrd[t] >> 5] = 0;
        }   // work
        tk = draw_front(ticket, t_end, &row_slot);     // its barriers also close this row's bitmap clean-up
    }
}

// The wavefront kernel for a pattern matrix B: the walk above with the mask row in a table of the wavefront's own.
// The table is 64 buckets of four columns, the bucket a multiplicative hash of the column, so a look-up is one
// 16-byte LDS read and four compares, without a loop.  A mask row goes in if no bucket overflows; three more
// multipliers are tried before the row is searched by bisection in memory instead, as are mask rows of more than
// SI_MASK_MAX entries (which sort to the other kernel's end of the list and only come here when this kernel gets
// that far).
constexpr int SI_MASK_MAX = 48;
constexpr int SI_TRIES = 4;
// a bucket read or cleared as one 16-byte access; may_alias, because the same words are also written one at a
// time by atomicCAS through an int pointer, and without it the compiler is free to reorder the two kinds
typedef int si_bucket __attribute__((ext_vector_type(4), may_alias));
struct BucketProbe {
    const int *tab;
    uint32_t mult;
    __device__ __forceinline__ static int bucket(int j, uint32_t mult)
    {
        return (int)((uint32_t)__umul24((uint32_t)j, mult) >> 26);      // __umul24 returns int: shift it as unsigned
    }
    __device__ __forceinline__ int one(int j) const
    {
        const si_bucket b = *reinterpret_cast<const si_bucket *>(tab + 4 * bucket(j, mult));
        return (b.x == j) | (b.y == j) | (b.z == j) | (b.w == j);
    }
    __device__ __forceinline__ int four(sg_i4u j) const { return one(j.x) + one(j.y) + one(j.z) + one(j.w); }
};
struct BisectProbe {
    const int32_t *m;       // the mask row, ascending
    int n;
    __device__ __forceinline__ int one(int j) const
    {
        int lo = 0, hi = n;
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (m[mid] < j)
                lo = mid + 1;
            else
                hi = mid;
        }
        return lo < n && m[lo] == j;
    }
    __device__ __forceinline__ int four(sg_i4u j) const { return one(j.x) + one(j.y) + one(j.z) + one(j.w); }
};

__global__ __launch_bounds__(SM_WAVES * 64) void spgemm_masked_sum_small_iso_kernel(
    const int64_t *__restrict__ Apos, const int32_t *__restrict__ Acrd, const double *__restrict__ Aval,
    const int64_t *__restrict__ Bpos, const int32_t *__restrict__ Bcrd, double biso,
    const int64_t *__restrict__ Mpos, const int32_t *__restrict__ Mcrd, unsigned long long *ticket, RowList list,
    double *__restrict__ rowsum)
{
    __shared__ __align__(16) int table[SM_WAVES][SM_SLOTS];
    const int lane = threadIdx.x & 63;
    int *tab = table[threadIdx.x >> 6];
    reinterpret_cast<si_bucket *>(tab)[lane] = si_bucket{-1, -1, -1, -1};
    int64_t t_first, t_end;
    list_range(list, 2, &t_first, &t_end);
    int take = SM_BATCH;
    for (;;) {
        // rows from the light end of the list, as spgemm_masked_sum_small_kernel draws them
        unsigned long long drawn = 0;
        if (lane == 0)
            drawn = atomicAdd(ticket, (unsigned long long)take << 32);
        const int64_t f = (int64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(drawn & 0xffffffffu));
        const int64_t b = (int64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(drawn >> 32));
        if (f + b >= t_end)
            break;
        const int nb = (int)(b + take < t_end - f ? take : t_end - f - b);      // what the front had not reached
        const int64_t taken = b + take;
        take = taken < t_end / 2 ? SM_BATCH : taken < t_end - t_end / 4 ? SM_BATCH / 4 : 1;
        // the rows of the batch and where they start and end in A and in the mask: one round trip for all of them
        int bi = 0;
        int64_t bas = 0, bae = 0, bms = 0, bme = 0;
        if (lane < nb) {
            bi = list.rows[t_end - 1 - (b + lane)];
            bas = Apos[bi];
            bae = Apos[bi + 1];
            bms = Mpos[bi];
            bme = Mpos[bi + 1];
        }
        for (int r = 0; r < nb; ++r) {
            const int i = __builtin_amdgcn_readlane(bi, r);
            const int64_t as = readlane_i64(bas, r), ae = readlane_i64(bae, r);
            const int64_t ms = readlane_i64(bms, r), me = readlane_i64(bme, r);
            if (as == ae || ms == me)
                continue;               // rowsum[i] keeps the zero the host put there
            const int mlen = (int)(me - ms < (int64_t)SI_MASK_MAX + 1 ? me - ms : SI_MASK_MAX + 1);
            bool hashed = false;
            uint32_t mult = 0;
            if (mlen <= SI_MASK_MAX) {
                const int j = lane < mlen ? Mcrd[ms + lane] : -1;
                static_assert(SI_MASK_MAX <= 64, "a lane holds one column of the mask row");
                for (int attempt = 0; attempt < SI_TRIES && !hashed; ++attempt) {
                    mult = attempt == 0 ? 0x9E3779u : attempt == 1 ? 0x85EBCBu : attempt == 2 ? 0xC2B2AFu : 0x27D4EBu;
                    bool placed = j < 0;
                    if (j >= 0) {
                        int *bk = tab + 4 * BucketProbe::bucket(j, mult);
#pragma unroll
                        for (int x = 0; x < 4; ++x)
                            if (!placed)
                                placed = atomicCAS(&bk[x], -1, j) == -1;
                    }
                    hashed = !__any(!placed);
                    if (!hashed)
                        reinterpret_cast<si_bucket *>(tab)[lane] = si_bucket{-1, -1, -1, -1};
                }
            }
            double part;
            if (hashed)
                part = iso_walk<1>(as, ae, Acrd, Aval, Bpos, Bcrd, biso, BucketProbe{tab, mult}, 0, lane);
            else
                part = iso_walk<1>(as, ae, Acrd, Aval, Bpos, Bcrd, biso, BisectProbe{Mcrd + ms, (int)(me - ms)}, 0, lane);
            part = wave_sum_f64(part);
            if (lane == 0)
                rowsum[i] = part;
            if (hashed)
                reinterpret_cast<si_bucket *>(tab)[lane] = si_bucket{-1, -1, -1, -1};
        }
    }
}

// whether all stored values of a matrix are one number (looked at once per matrix)
__global__ void csr_values_differ(int64_t nnz, const double *__restrict__ val, int *__restrict__ flag)
{
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p < nnz && val[p] != val[0])
        *flag = 1;
}

// ---------------------------------------------------------------------------
// CSR .* CSR -> CSR, one lane per row, two-pointer merge of the sorted rows
// (lib/Conversion/IndexTreeToSCF/IndexTreeToSCF.cpp:864-1053).
// ---------------------------------------------------------------------------
template <bool FILL>
__global__ void eltwise_mult_kernel(int64_t nrows, const int64_t *__restrict__ Apos,
                                    const int32_t *__restrict__ Acrd, const double *__restrict__ Aval,
                                    const int64_t *__restrict__ Bpos, const int32_t *__restrict__ Bcrd,
                                    const double *__restrict__ Bval, int64_t *__restrict__ rowcount,
                                    const int64_t *__restrict__ Cpos, int32_t *__restrict__ Ccrd,
                                    double *__restrict__ Cval)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nrows)
        return;
    int64_t p = Apos[i], q = Bpos[i];
    const int64_t pe = Apos[i + 1], qe = Bpos[i + 1];
    int64_t n = 0;
    int64_t o = FILL ? Cpos[i] : 0;
    while (p < pe && q < qe) {
        const int ca = Acrd[p], cb = Bcrd[q];
        if (ca == cb) {
            if (FILL) {
                Ccrd[o] = ca;
                Cval[o] = Aval[p] * Bval[q];
                ++o;
            }
            ++n;
        }
        p += (ca <= cb);
        q += (cb <= ca);
    }
    if (!FILL)
        rowcount[i] = n;
}

// CSR (op) Dense, op = * for the plain elementwise product and any other COMET_OP_* for the monoid forms
// A @(op) B of test/integration/semiring/eltwise_monoid*_COOxDense_oCOO.ta: the stored entries of A combined
// with the dense values under them.  TO_DENSE writes them into a dense
// output at their positions and leaves every other element as it was (the nest only visits the entries of
// A, test/integration/ops/eltwise_mult_CSRxDense_oDense.ta); otherwise they become the values of a CSR with
// A's structure (eltwise_mult_CSRxDense_oCSR.ta).
template <bool TO_DENSE>
__global__ void eltwise_mult_dense_kernel(int64_t nrows, const int64_t *__restrict__ pos,
                                          const int32_t *__restrict__ crd, const double *__restrict__ val,
                                          const double *__restrict__ D, int64_t ldd, double *__restrict__ out,
                                          int64_t ldo, int op)
{
    // one 16-lane group per row
    const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 4;
    if (i >= nrows)
        return;
    for (int64_t p = pos[i] + (threadIdx.x & 15); p < pos[i + 1]; p += 16) {
        const double v = semiring_mult(op, val[p], D[i * ldd + crd[p]]);
        if (TO_DENSE)
            out[i * ldo + crd[p]] = v;
        else
            out[p] = v;
    }
}

// ------------------------------------------------------------------ host side
// ---------------------------------------------------------------------------
// Masked products as dot products over the mask (the reference's masked Gustavson nest,
// lib/Conversion/IndexTreeToSCF/IndexTreeToSCF.cpp:1083-1148 and :1327-1448, walks every product of row i and tests
// its column against the mask row's mark array; C keeps the mask's entries that received a product, in mask order -
// what comes out here is the same set and, per entry, the same sum).  C<M>[i][j] = sum over k of A[i][k] * B[k][j] is the dot product of
// row i of A and column j of B; walking the products of row i (every entry of every B_k, k in A_i) costs |B_k|
// look-ups per entry of A_i whatever the mask holds, the dot product of a stored pair (i, j) costs the shorter of
// its two lists when that one is streamed against a table of the longer one.  So the pairs of the mask are split
// by which list is longer.  One kernel serves both halves: a workgroup takes a row x of a matrix of pairs P,
// puts the list T_x into its table, and for the pairs (x, y) of P_x that are its to do streams the list L_y
// through the table.
//   the row's half:     P = M,   T = A (rows),            L = B^T (columns of B);  pair (i, j) when |B^T_j| <= |A_i|
//   the column's half:  P = M^T, T = B^T (columns of B),  L = A (rows);            pair (j, i) when |A_i| < |B^T_j|
// The table is a bitmap over k in LDS with the number of set bits before every eighth word, so that a hit knows
// its rank in T_x and with it where the value lies (a list in the table must not hold a column twice).  A pair's
// products are added into a slot of LDS that belongs to the wavefront and the pair (64 pairs per wavefront at a
// time) and leave, with the flag that says whether there was any, when the wavefront is through with its 64.
// ---------------------------------------------------------------------------
struct DotHit {
    int hit;
    double prod;
};
constexpr int DT_GROUP = 16;         // bitmap words per count
constexpr int DT_WPT = 32;           // consecutive bitmap words a thread counts: SG_T * DT_WPT * 32 = 2^20 columns at most
// The table of a list of at most SG_HASH_FILL entries is a hash table instead, key k + 1 and the value, in the same
// LDS: nothing to count, and building and clearing it costs by the length of the list, not of the bitmap.
// Words of LDS in front of the wavefronts' sums: the bitmap (one padding word after every 32, so that a thread's
// 32 consecutive words lie in 32 banks) and the counts, or the hash table's keys and values, whichever is more
constexpr int dot_bitmap_words(int words) { return words + words / 32 + words / DT_GROUP; }
constexpr int dot_table_words(int words)
{
    return ((dot_bitmap_words(words) > 3 * SG_HASH_SLOTS ? dot_bitmap_words(words) : 3 * SG_HASH_SLOTS) + 1) & ~1;
}
constexpr size_t dot_lds_bytes(int words)
{
    return (size_t)dot_table_words(words) * 4 + (size_t)SG_WAVES * 64 * (8 + 4);
}
static_assert(dot_lds_bytes(SG_T * DT_WPT) <= 160 * 1024 - 256, "the table of 2^20 columns fits LDS");
// the fp64 regions of the dot-product kernel: the hash table's values SG_HASH_SLOTS words in, the wavefronts' sums
// dot_table_words(words) words in, for every table size the host can ask for (a multiple of DT_WPT words)
constexpr bool dot_fp64_regions_aligned()
{
    if (SG_HASH_SLOTS % 2 != 0)
        return false;
    for (int w = DT_WPT; w <= SG_T * DT_WPT; w += DT_WPT)
        if (dot_table_words(w) % 2 != 0)
            return false;
    return true;
}
static_assert(dot_fp64_regions_aligned(), "an fp64 region of the dot-product kernel's LDS is not 8-byte aligned");

// The pairs [ms, me) of one row of P, dealt to the wavefronts like the entries of a row of A in
// for_each_product_impl (the walk of a turn and its one-turn-late visits are the same); keep(y, len) says whether
// a pair is this half's; f gets the pair's slot in the wavefront's batch; done(base, cnt, kept) ends a batch.
// With VALUES the entries' values are loaded with their columns and handed to mid: in these products a fifth of the
// look-ups hit, so nearly every cache line of the values is needed anyway, and fetched only for the hits they would
// be a second trip to memory behind the first.
// Without VALUES only whether a pair meets a product is asked, and decided(t) says that pair t of the wavefront's
// batch already has: the rest of its list is then left out (a long list is through after a turn or two).
template <bool VALUES, typename KEEP, typename PRE, typename MID, typename F, typename DONE, typename DECIDED>
__device__ inline void for_each_pair(int64_t ms, int64_t me, const int32_t *__restrict__ Pcrd,
                                     const int64_t *__restrict__ Lpos, const int32_t *__restrict__ Lcrd,
                                     const double *__restrict__ Lval, KEEP keep, PRE pre, MID mid, F f, DONE done,
                                     DECIDED decided)
{
    using T1 = decltype(pre(0));
    using T2 = decltype(mid(0, 0.0, T1()));
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int quarter = lane >> 4, sub = lane & 15;
    constexpr int NP = FEP_LONG_LOADS > FEP_SHORT_LOADS ? FEP_LONG_LOADS : FEP_SHORT_LOADS;
    bool w_ok[NP];
    int w_t[NP];
    T2 w_md[NP];
#pragma unroll
    for (int x = 0; x < NP; ++x)
        w_ok[x] = false;
    const auto visit_pending = [&]() {
#pragma unroll
        for (int x = 0; x < NP; ++x)
            if (w_ok[x])
                f(w_t[x], w_md[x]);
#pragma unroll
        for (int x = 0; x < NP; ++x)
            w_ok[x] = false;
    };
    const auto turn = [&](auto n_tag, const bool *ok, const int *k, const double *v, int t) {
        constexpr int N = decltype(n_tag)::value;
        T1 tk[N];
#pragma unroll
        for (int x = 0; x < N; ++x)
            tk[x] = ok[x] ? pre(k[x]) : T1();
        visit_pending();
#pragma unroll
        for (int x = 0; x < N; ++x) {
            w_ok[x] = ok[x];
            w_t[x] = t;
            w_md[x] = ok[x] ? mid(k[x], v[x], tk[x]) : T2();
        }
    };
    for (int64_t base = ms + wave; base < me; base += (int64_t)SG_WAVES * 64) {
        const int64_t left = (me - base + SG_WAVES - 1) / SG_WAVES;     // my pairs from here on
        const int cnt = (int)(left < 64 ? left : 64);
        int64_t bs = 0, be = 0;
        bool kept = false;
        if (lane < cnt) {
            const int y = Pcrd[base + (int64_t)lane * SG_WAVES];
            bs = Lpos[y];
            be = Lpos[y + 1];
            kept = keep(y, be - bs);
            if (!kept)
                be = bs;
        }
        unsigned long long big = __ballot(be - bs >= FEP_SHORT);
        unsigned long long todo = __ballot(bs < be && be - bs < FEP_SHORT);
        while (big) {
            const int t = __builtin_ctzll(big);
            big &= big - 1;
            const int64_t s = readlane_i64(bs, t), len = readlane_i64(be, t) - s;
            int64_t o = lane;
            if (len >= 64 * FEP_LONG_LOADS) {
                bool all[FEP_LONG_LOADS];
                int k[FEP_LONG_LOADS];
                double v[FEP_LONG_LOADS];
#pragma unroll
                for (int x = 0; x < FEP_LONG_LOADS; ++x) {
                    all[x] = true;
                    k[x] = Lcrd[s + o + 64 * x];
                    v[x] = VALUES ? Lval[s + o + 64 * x] : 0.0;
                }
                bool enough = false;
                for (int64_t full = 64 * FEP_LONG_LOADS; full + 64 * FEP_LONG_LOADS <= len;
                     full += 64 * FEP_LONG_LOADS) {
                    if (!VALUES && decided(t)) {        // what earlier turns found (a turn's visits come one turn late)
                        enough = true;
                        break;
                    }
                    int kn[FEP_LONG_LOADS];
                    double vn[FEP_LONG_LOADS];
#pragma unroll
                    for (int x = 0; x < FEP_LONG_LOADS; ++x) {
                        kn[x] = Lcrd[s + o + 64 * (FEP_LONG_LOADS + x)];
                        vn[x] = VALUES ? Lval[s + o + 64 * (FEP_LONG_LOADS + x)] : 0.0;
                    }
                    turn(std::integral_constant<int, FEP_LONG_LOADS>(), all, k, v, t);
#pragma unroll
                    for (int x = 0; x < FEP_LONG_LOADS; ++x) {
                        k[x] = kn[x];
                        v[x] = vn[x];
                    }
                    o += 64 * FEP_LONG_LOADS;
                }
                turn(std::integral_constant<int, FEP_LONG_LOADS>(), all, k, v, t);
                o += 64 * FEP_LONG_LOADS;
                if (enough)
                    o = len;
            }
            if (o < len && (VALUES || !decided(t))) {
                bool ok[FEP_LONG_LOADS];
                int k[FEP_LONG_LOADS];
                double v[FEP_LONG_LOADS];
#pragma unroll
                for (int x = 0; x < FEP_LONG_LOADS; ++x)
                    ok[x] = o + 64 * x < len;
#pragma unroll
                for (int x = 0; x < FEP_LONG_LOADS; ++x)
                    k[x] = ok[x] ? Lcrd[s + o + 64 * x] : 0;
#pragma unroll
                for (int x = 0; x < FEP_LONG_LOADS; ++x)
                    v[x] = VALUES && ok[x] ? Lval[s + o + 64 * x] : 0.0;
                turn(std::integral_constant<int, FEP_LONG_LOADS>(), ok, k, v, t);
            }
        }
        while (todo) {
            int pick = -1;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int t = todo ? __builtin_ctzll(todo) : -1;
                todo = todo ? (todo & (todo - 1)) : 0;
                pick = quarter == g ? t : pick;
            }
            const int src = pick < 0 ? lane : pick;
            const int64_t s = ((int64_t)__shfl((int)(bs >> 32), src, 64) << 32) |
                              (uint32_t)__shfl((int)(bs & 0xffffffff), src, 64);
            const int64_t e = ((int64_t)__shfl((int)(be >> 32), src, 64) << 32) |
                              (uint32_t)__shfl((int)(be & 0xffffffff), src, 64);
            bool ok[FEP_SHORT_LOADS];
            int k[FEP_SHORT_LOADS];
            double v[FEP_SHORT_LOADS];
#pragma unroll
            for (int x = 0; x < FEP_SHORT_LOADS; ++x)
                ok[x] = pick >= 0 && s + sub + 16 * x < e;
#pragma unroll
            for (int x = 0; x < FEP_SHORT_LOADS; ++x)
                k[x] = ok[x] ? Lcrd[s + sub + 16 * x] : 0;
#pragma unroll
            for (int x = 0; x < FEP_SHORT_LOADS; ++x)
                v[x] = VALUES && ok[x] ? Lval[s + sub + 16 * x] : 0.0;
            turn(std::integral_constant<int, FEP_SHORT_LOADS>(), ok, k, v, src);
        }
        visit_pending();
        done(base, cnt, kept);
    }
}

// strict: a pair is kept when its streamed list is shorter than the table's (otherwise: not longer).  [xlo, xhi):
// the pairs' other index must lie in it (the rows of M being computed, for the column's half).  perm: where pair p
// of P lies in the row-major order of the mask (nullptr: at p); out0 is taken off either.
// SEMI: another semiring than plus-times (reduce plus, min or max; `any` keeps the place of a product in B, which
// this form does not have): a product is mult(a, b) with a the entry of A - the table's in the row's half, the
// streamed one in the column's (swapped) - and a pair's slot holds a sum or the key of a minimum or maximum.
template <bool VALUES, bool SEMI>
__global__ __launch_bounds__(SG_T) void spgemm_dot_kernel(
    int64_t row_begin, const int64_t *__restrict__ Tpos, const int32_t *__restrict__ Tcrd,
    const double *__restrict__ Tval, const int64_t *__restrict__ Ppos, const int32_t *__restrict__ Pcrd,
    const int64_t *__restrict__ Lpos, const int32_t *__restrict__ Lcrd, const double *__restrict__ Lval,
    const double *__restrict__ perm, int64_t out0, int strict, int64_t xlo, int64_t xhi, int words,
    unsigned long long *ticket, RowList list, double *__restrict__ pair_val, uint8_t *__restrict__ pair_hit,
    int reduce_op, int mult_op, int swapped)
{
    __shared__ int64_t row_slot;
    __shared__ int wave_tot[SG_WAVES];
    uint32_t *bm = sg_dyn_lds;
    uint32_t *cnt_before = bm + words + words / 32;    // [words / DT_GROUP]
    uint32_t *hkey = sg_dyn_lds;                       // [SG_HASH_SLOTS], over the bitmap
    double *hval = reinterpret_cast<double *>(sg_dyn_lds + SG_HASH_SLOTS);        // [SG_HASH_SLOTS]
    const int table_words = dot_table_words(words);
    double *wacc = reinterpret_cast<double *>(sg_dyn_lds + table_words);           // [SG_WAVES][64]
    int *whit = reinterpret_cast<int *>(wacc + SG_WAVES * 64);                     // [SG_WAVES][64]
    const BmAddr ad{5};
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    for (int w = threadIdx.x; w < table_words; w += SG_T)
        sg_dyn_lds[w] = 0;
    wacc[threadIdx.x] = 0.0;
    whit[threadIdx.x] = 0;
    lds_barrier();
    bool values_left = false;       // a hash table's values lie where bitmap words are: cleared before the next bitmap
    int64_t t_first, t_end;
    list_range(list, 2, &t_first, &t_end);
    int64_t tk = draw_row<true>(ticket, t_first, &row_slot);
    while (tk < t_end) {
        const int64_t x = row_begin + list.rows[tk];
        const int64_t ts = Tpos[x], te = Tpos[x + 1];
        const int64_t ps = Ppos[x], pe = Ppos[x + 1];
        const int64_t tlen = te - ts;
        const auto keep = [&](int y, int64_t len) {
            return len > 0 && (strict ? len < tlen : len <= tlen) && y >= xlo && y < xhi;
        };
        const auto add = [&](int t, DotHit h) {
            if (h.hit) {
                whit[wave * 64 + t] = 1;
                if constexpr (VALUES && SEMI) {
                    if (reduce_op == SR_PLUS)
                        __hip_atomic_fetch_add(&wacc[wave * 64 + t], h.prod, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    else
                        __hip_atomic_fetch_max(reinterpret_cast<unsigned long long *>(&wacc[wave * 64 + t]),
                                               reduce_op == SR_MIN ? ~f64_key(h.prod) : f64_key(h.prod), __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_WORKGROUP);
                } else if constexpr (VALUES) {
                    __hip_atomic_fetch_add(&wacc[wave * 64 + t], h.prod, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
            }
        };
        // tv: the table's value, lv: the streamed entry's
        const auto product = [&](double tv, double lv) {
            if constexpr (SEMI)
                return swapped ? semiring_mult(mult_op, lv, tv) : semiring_mult(mult_op, tv, lv);
            else
                return tv * lv;
        };
        // (uniform: t is; a wavefront's own LDS operations keep their order)
        const auto decided = [&](int t) { return __builtin_amdgcn_readfirstlane(whit[wave * 64 + t]) != 0; };
        const auto done = [&](int64_t base, int cnt, bool kept) {
            // the slots belong to this wavefront, which has issued all its adds: LDS keeps a wavefront's order
            if (lane < cnt && kept) {
                const int64_t p = base + (int64_t)lane * SG_WAVES;
                const int64_t at = (perm ? (int64_t)perm[p] : p) - out0;
                pair_hit[at] = (uint8_t)whit[wave * 64 + lane];
                if constexpr (VALUES && SEMI)
                    pair_val[at] = semiring_lds_value(reinterpret_cast<unsigned long long *>(wacc)[wave * 64 + lane],
                                                      reduce_op, mult_op, 0, nullptr, nullptr);
                else if constexpr (VALUES)
                    pair_val[at] = wacc[wave * 64 + lane];
            }
            wacc[wave * 64 + lane] = 0.0;
            whit[wave * 64 + lane] = 0;
        };
        if (ts != te && ps != pe && tlen <= SG_HASH_FILL) {
            for (int64_t t = ts + threadIdx.x; t < te; t += SG_T) {
                const int k = Tcrd[t];
                const uint32_t key = (uint32_t)k + 1u;
                uint32_t sl = sg_hash_slot(k);
                for (;;) {
                    const uint32_t old = atomicCAS(&hkey[sl], 0u, key);
                    if (old == 0u)
                        break;
                    sl = (sl + 1) & (SG_HASH_SLOTS - 1);
                }
                if constexpr (VALUES)
                    hval[sl] = Tval[t];
            }
            values_left = VALUES;
            lds_barrier();
            for_each_pair<VALUES>(ps, pe, Pcrd, Lpos, Lcrd, Lval, keep,
                [&](int k) { return hkey[sg_hash_slot(k)]; },
                [&](int k, double lv, uint32_t k0) {
                    DotHit h{0, 0.0};
                    if (k0 != 0u) {
                        uint32_t sl = sg_hash_slot(k);
                        uint32_t key = k0;
                        while (key != 0u && key != (uint32_t)k + 1u) {
                            sl = (sl + 1) & (SG_HASH_SLOTS - 1);
                            key = hkey[sl];
                        }
                        if (key != 0u) {
                            h.hit = 1;
                            if constexpr (VALUES)
                                h.prod = product(hval[sl], lv);
                        }
                    }
                    return h;
                }, add, done, decided);
            lds_barrier();
            for (int sl = threadIdx.x; sl < SG_HASH_SLOTS; sl += SG_T)
                hkey[sl] = 0u;
        } else if (ts != te && ps != pe) {
            if (values_left) {
                for (int w = SG_HASH_SLOTS + threadIdx.x; w < 3 * SG_HASH_SLOTS; w += SG_T)
                    sg_dyn_lds[w] = 0;
                values_left = false;
                lds_barrier();
            }
            for (int64_t t = ts + threadIdx.x; t < te; t += SG_T) {
                const int k = Tcrd[t];
                atomicOr(&bm[ad.word(k)], ad.bit(k));
            }
            lds_barrier();
            {   // bits before every group of words: a thread counts DT_WPT consecutive words
                const int w0 = (int)threadIdx.x * DT_WPT;
                int mine = 0;
                if (w0 < words) {
#pragma unroll
                    for (int c = 0; c < DT_WPT; ++c)
                        mine += __popc(bm[w0 + c + (w0 >> 5)]);
                }
                const int inc = wave_inclusive_scan(mine);
                if (lane == 63)
                    wave_tot[wave] = inc;
                lds_barrier();
                const int tots = wave_inclusive_scan(lane < SG_WAVES ? wave_tot[lane] : 0);
                int run = (wave ? __builtin_amdgcn_readlane(tots, wave - 1) : 0) + inc - mine;
                if (w0 < words) {
#pragma unroll
                    for (int c = 0; c < DT_WPT; ++c) {
                        if (c % DT_GROUP == 0)
                            cnt_before[(w0 + c) / DT_GROUP] = (uint32_t)run;
                        run += __popc(bm[w0 + c + (w0 >> 5)]);
                    }
                }
                lds_barrier();
            }
            for_each_pair<VALUES>(ps, pe, Pcrd, Lpos, Lcrd, Lval, keep,
                [&](int k) { return bm[ad.word(k)]; },
                [&](int k, double lv, uint32_t word) {
                    DotHit h{0, 0.0};
                    if (word & ad.bit(k)) {
                        h.hit = 1;
                        if constexpr (VALUES) {
                            const int w = k >> 5, wg = w & ~(DT_GROUP - 1);
                            int rank = (int)cnt_before[w / DT_GROUP] + __popc(word & (ad.bit(k) - 1u));
                            for (int v = wg; v < w; ++v)
                                rank += __popc(bm[v + (v >> 5)]);
                            h.prod = product(Tval[ts + rank], lv);
                        }
                    }
                    return h;
                }, add, done, decided);
            lds_barrier();
            for (int64_t t = ts + threadIdx.x; t < te; t += SG_T)
                bm[ad.word(Tcrd[t])] = 0;
        }
        tk = draw_row<true>(ticket, t_first, &row_slot);      // its barriers also close this row's clean-up
    }
}

// rowcount[i - rb] = stored pairs of mask row i that met a product
__global__ __launch_bounds__(256) void spgemm_dot_count(int64_t rb, int64_t re, const int64_t *__restrict__ Mpos,
                                                        const uint8_t *__restrict__ pair_hit,
                                                        int64_t *__restrict__ rowcount)
{
    const int64_t i = rb + (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= re)
        return;
    const int lane = threadIdx.x & 63;
    const int64_t out0 = Mpos[rb];
    int n = 0;
    for (int64_t p = Mpos[i] + lane; p < Mpos[i + 1]; p += 64)
        n += pair_hit[p - out0];
    n = wave_sum_i32(n);
    if (lane == 0)
        rowcount[i - rb] = n;
}

// the pairs that met a product, in the order of the mask row, to the place Cpos gives the row
__global__ __launch_bounds__(256) void spgemm_dot_compact(int64_t rb, int64_t re, const int64_t *__restrict__ Mpos,
                                                          const int32_t *__restrict__ Mcrd,
                                                          const double *__restrict__ pair_val,
                                                          const uint8_t *__restrict__ pair_hit,
                                                          const int64_t *__restrict__ Cpos, int32_t *__restrict__ Ccrd,
                                                          double *__restrict__ Cval)
{
    const int64_t i = rb + (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= re)
        return;
    const int lane = threadIdx.x & 63;
    const int64_t in0 = Mpos[rb];
    int64_t at = Cpos[i] - Cpos[rb];
    for (int64_t base = Mpos[i]; base < Mpos[i + 1]; base += 64) {
        const int64_t p = base + lane;
        const bool hit = p < Mpos[i + 1] && pair_hit[p - in0];
        const unsigned long long m = __ballot(hit);
        if (hit) {
            const int64_t o = at + __popcll(m & ((1ull << lane) - 1ull));
            Ccrd[o] = Mcrd[p];
            Cval[o] = pair_val[p - in0];
        }
        at += __popcll(m);
    }
}

// flag[0] |= 1 when a row holds a column twice (rows are sorted); a wavefront per row
__global__ __launch_bounds__(256) void csr_find_duplicates(int64_t nrows, const int64_t *__restrict__ pos,
                                                           const int32_t *__restrict__ crd, int *__restrict__ flag)
{
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= nrows)
        return;
    bool twice = false;
    for (int64_t p = pos[r] + (threadIdx.x & 63); p + 1 < pos[r + 1]; p += 64)
        twice = twice || crd[p] == crd[p + 1];
    if (twice)
        atomicOr(flag, 1);
}

__global__ void fill_iota_f64(int64_t n, double *__restrict__ out)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        out[i] = (double)i;
}

struct SgScratch {
    Workspace ticket;     // one 64-bit row counter
    Workspace rowcount;   // int64[nrows] / double[nrows]
    Workspace gbm;        // global bitmaps (only when the bitmap does not fit LDS)
    Workspace gmask;      // global mask bitmaps (masked numeric)
    Workspace slabs;      // dense accumulators, zero between calls
    Workspace dense_rows;     // DenseRow[] and before[] of spgemm_numeric_dense_blocks_kernel
    Workspace dense_before;
    Workspace gave_up;        // its flag, zero between calls
};
static SgScratch g_sg;

struct SgGeom {
    int logW;
    bool lds;
    int groups;
    size_t lds_bytes;
    size_t bm_words;      // words per workgroup bitmap
};

static int sg_geometry(int64_t ncols, SgGeom *g)
{
    const int64_t words = ceil_div(ncols > 0 ? ncols : 1, 32);
    int logW = 0;
    while (((int64_t)SG_T << logW) < words)
        ++logW;
    if (logW > 20)
        return set_error(COMET_HIP_ERR_SIZE, "too many columns (%lld)", (long long)ncols);
    g->logW = logW;
    g->lds = (1 << logW) <= SG_LDS_MAX_W;
    g->bm_words = (size_t)SG_T * ((size_t)(1 << logW) + 1);
    g->lds_bytes = g->lds ? g->bm_words * sizeof(uint32_t) : 0;
    g->groups = num_cus() > 0 ? num_cus() : 256;
    if (g->lds && g->lds_bytes <= 48 * 1024)
        g->groups *= 2;          // two workgroups of 16 wavefronts fit a CU when the bitmap is small
    return COMET_HIP_OK;
}

template <typename K>
static int sg_allow_lds(K kernel, size_t bytes)
{
    if (bytes > 0)
        COMET_HIPCHK(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
    return COMET_HIP_OK;
}

static int sg_reset_ticket()
{
    COMET_CHK(g_sg.ticket.ensure(sizeof(unsigned long long), false));
    COMET_HIPCHK(hipMemsetAsync(g_sg.ticket.ptr, 0, sizeof(unsigned long long), stream()));
    return COMET_HIP_OK;
}

static int check_product_shapes(const Csr *a, const Csr *b, const Csr *m, const char *who)
{
    if (a->ncols != b->nrows)
        return set_error(COMET_HIP_ERR_ARG, "%s: A is %lld x %lld but B is %lld x %lld", who, (long long)a->nrows,
                         (long long)a->ncols, (long long)b->nrows, (long long)b->ncols);
    if (m && (m->nrows != a->nrows || m->ncols != b->ncols))
        return set_error(COMET_HIP_ERR_ARG, "%s: mask is %lld x %lld, product is %lld x %lld", who,
                         (long long)m->nrows, (long long)m->ncols, (long long)a->nrows, (long long)b->ncols);
    return COMET_HIP_OK;
}

// keys that order rows by descending products; rows without products sort to the very end
// With a mask (Mpos, already offset to the first row of the list), the rows whose mask row holds more than `fill`
// entries sort in front of all others (keys below 2^61), whatever their number of products.
__global__ void sg_row_keys(int64_t n, const int64_t *__restrict__ rowprod, const int64_t *__restrict__ Mpos,
                            int64_t fill, uint64_t *__restrict__ keys, uint32_t *__restrict__ idx)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r < n) {
        const int64_t p = rowprod[r];
        uint64_t key = p > 0 ? (uint64_t)((1ll << 62) - p) : ~0ull >> 1;
        if (Mpos && p > 0 && Mpos[r + 1] - Mpos[r] > fill)
            key = (uint64_t)((1ll << 61) - (p < (1ll << 61) ? p : (1ll << 61) - 1));
        keys[r] = key;
        idx[r] = (uint32_t)r;
    }
}

// bounds[0] = rows with >= threshold products, bounds[1] = rows with any, bounds[2] = rows with >= wide products,
// in the sorted key array
__global__ void sg_row_bounds(int64_t n, const uint64_t *__restrict__ keys, int64_t threshold, int64_t wide,
                              int64_t *__restrict__ bounds)
{
    if (threadIdx.x > 2 || blockIdx.x > 0)
        return;
    // first key that is larger than the limit: keys ascend as products descend
    const uint64_t limit = threadIdx.x == 1 ? (uint64_t)((1ll << 62) - 1)
                                            : (uint64_t)((1ll << 62) - (threadIdx.x == 0 ? threshold : wide));
    int64_t lo = 0, hi = n;
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if (keys[mid] <= limit)
            lo = mid + 1;
        else
            hi = mid;
    }
    bounds[threadIdx.x] = lo;
}

struct SgRowLists {
    Workspace rowprod, keys_in, keys_out, idx_in, idx_out, bounds;
};
static SgRowLists g_rl;

// Products per row of rows [rb, re) of A*B and the list of those rows by descending products.
struct SgPairFilter {          // see spgemm_row_products
    const Csr *towner = nullptr;        // tpos = towner->pos
    int strict = 0;
    int64_t xlo = 0, xhi = 0;
};
// The list depends on the two structures, the range and the thresholds only: it is kept in A's handle and found
// again by the uids of the matrices it was made from (a matrix gets a new uid when it is invalidated), so a
// product that is taken again, or taken in row blocks, sorts nothing.  COMET_HIP_SPGEMM_NO_LIST_CACHE turns the
// keeping off (the tests compare both).
constexpr size_t SG_ROW_LISTS_KEPT = 24;
static int sg_row_list(const Csr *a, const Csr *b, int64_t rb, int64_t re, int64_t dense_threshold,
                       int64_t wide_threshold, RowList *out, const Csr *long_mask = nullptr,
                       int64_t mask_fill = 0, SgPairFilter filter = SgPairFilter())
{
    const int64_t n = re - rb;
    static const bool keep = getenv("COMET_HIP_SPGEMM_NO_LIST_CACHE") == nullptr;
    Csr *owner = const_cast<Csr *>(a);
    RowListEntry key;
    key.b_uid = b->uid;
    key.mask_uid = long_mask ? long_mask->uid : 0;
    key.filter_uid = filter.towner ? filter.towner->uid : 0;
    key.rb = rb;
    key.re = re;
    key.dense_threshold = dense_threshold;
    key.wide_threshold = wide_threshold;
    key.mask_fill = mask_fill;
    key.xlo = filter.xlo;
    key.xhi = filter.xhi;
    key.strict = filter.strict;
    if (keep)
        for (const RowListEntry &e : owner->row_lists)
            if (e.b_uid == key.b_uid && e.mask_uid == key.mask_uid && e.filter_uid == key.filter_uid && e.rb == rb &&
                e.re == re && e.dense_threshold == dense_threshold && e.wide_threshold == wide_threshold &&
                e.mask_fill == mask_fill && e.xlo == key.xlo && e.xhi == key.xhi && e.strict == key.strict) {
                out->rows = e.rows;
                out->bounds = e.bounds;
                return COMET_HIP_OK;
            }
    COMET_CHK(g_rl.rowprod.ensure(sizeof(int64_t) * (size_t)n, false));
    COMET_CHK(g_rl.keys_in.ensure(8 * (size_t)n, false));
    COMET_CHK(g_rl.keys_out.ensure(8 * (size_t)n, false));
    COMET_CHK(g_rl.idx_in.ensure(4 * (size_t)n, false));
    COMET_CHK(g_rl.idx_out.ensure(4 * (size_t)n, false));
    COMET_CHK(g_rl.bounds.ensure(24, false));
    int64_t *rowprod = (int64_t *)g_rl.rowprod.ptr;
    {
        KernelTimer t("spgemm_row_products");
        spgemm_row_products<<<dim3((unsigned)ceil_div(n, 4)), dim3(256), 0, stream()>>>(
            rb, re, a->pos, a->crd, b->pos, rowprod, filter.towner ? filter.towner->pos : nullptr, filter.strict,
            filter.xlo, filter.xhi);
        sg_row_keys<<<dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, stream()>>>(
            n, rowprod, long_mask ? long_mask->pos + rb : nullptr, mask_fill, (uint64_t *)g_rl.keys_in.ptr,
            (uint32_t *)g_rl.idx_in.ptr);
    }
    COMET_HIPCHK(hipGetLastError());
    COMET_CHK(sort_pairs_u64_u32((const uint64_t *)g_rl.keys_in.ptr, (uint64_t *)g_rl.keys_out.ptr,
                                 (const uint32_t *)g_rl.idx_in.ptr, (uint32_t *)g_rl.idx_out.ptr, n, 63));
    sg_row_bounds<<<dim3(1), dim3(64), 0, stream()>>>(n, (const uint64_t *)g_rl.keys_out.ptr, dense_threshold,
                                                      wide_threshold, (int64_t *)g_rl.bounds.ptr);
    COMET_HIPCHK(hipGetLastError());
    out->rows = (const int32_t *)g_rl.idx_out.ptr;
    out->bounds = (const int64_t *)g_rl.bounds.ptr;
    if (keep && n > 0) {
        // a copy of its own; failing to get the memory only means that the list is built again next time
        if (owner->row_lists.size() >= SG_ROW_LISTS_KEPT) {
            COMET_HIPCHK(hipStreamSynchronize(stream()));        // a kernel may still be reading the oldest one
            (void)hipFree(owner->row_lists.front().rows);
            (void)hipFree(owner->row_lists.front().bounds);
            owner->row_lists.erase(owner->row_lists.begin());
        }
        if (hipMalloc((void **)&key.rows, 4 * (size_t)n) != hipSuccess ||
            hipMalloc((void **)&key.bounds, 24) != hipSuccess) {
            (void)hipGetLastError();
            (void)hipFree(key.rows);
            return COMET_HIP_OK;
        }
        COMET_HIPCHK(hipMemcpyAsync(key.rows, g_rl.idx_out.ptr, 4 * (size_t)n, hipMemcpyDeviceToDevice, stream()));
        COMET_HIPCHK(hipMemcpyAsync(key.bounds, g_rl.bounds.ptr, 24, hipMemcpyDeviceToDevice, stream()));
        owner->row_lists.push_back(key);
        out->rows = key.rows;
        out->bounds = key.bounds;
    }
    return COMET_HIP_OK;
}

constexpr int64_t SG_NO_DENSE = 1ll << 61;     // a threshold no row reaches: every row stays on the slab path

static int dot_form_fits(const Csr *a, const Csr *b, const Csr *m, bool *fits);
static int dot_pairs(const Csr *a, const Csr *b, const Csr *m, int64_t rb, int64_t re, bool values, double **pair_val,
                     uint8_t **pair_hit, int reduce_op = COMET_SR_PLUS, int mult_op = COMET_OP_TIMES);

static int symbolic_counts(const Csr *a, const Csr *b, const Csr *m, int64_t *rowcount)
{
    bool dots = false;
    COMET_CHK(dot_form_fits(a, b, m, &dots));
    if (dots) {         // a masked product: which stored pairs of the mask meet a product
        double *pair_val = nullptr;
        uint8_t *pair_hit = nullptr;
        COMET_CHK(dot_pairs(a, b, m, 0, a->nrows, false, &pair_val, &pair_hit));
        KernelTimer t("spgemm_symbolic_dot_count");
        spgemm_dot_count<<<dim3((unsigned)ceil_div(a->nrows, 4)), dim3(256), 0, stream()>>>(0, a->nrows, m->pos, pair_hit,
                                                                                            rowcount);
        COMET_HIPCHK(hipGetLastError());
        return COMET_HIP_OK;
    }
    SgGeom g;
    COMET_CHK(sg_geometry(b->ncols, &g));
    COMET_CHK(sg_reset_ticket());
    RowList list;
    COMET_CHK(sg_row_list(a, b, 0, a->nrows, SG_NO_DENSE, SG_NO_DENSE, &list));
    COMET_HIPCHK(hipMemsetAsync(rowcount, 0, sizeof(int64_t) * (size_t)a->nrows, stream()));
    uint32_t *gbm = nullptr;
    if (!g.lds) {
        COMET_CHK(g_sg.gbm.ensure(sizeof(uint32_t) * g.bm_words * (size_t)g.groups, true));
        gbm = (uint32_t *)g_sg.gbm.ptr;
    }
    const dim3 grid((unsigned)g.groups), block(SG_T);
#define LAUNCH_SYM(L, M)                                                                                   \
    do {                                                                                                   \
        COMET_CHK(sg_allow_lds(spgemm_symbolic_kernel<L, M>, g.lds_bytes));                                \
        KernelTimer t(M ? "spgemm_symbolic_masked" : "spgemm_symbolic");                                   \
        spgemm_symbolic_kernel<L, M><<<grid, block, g.lds_bytes, stream()>>>(                              \
            a->nrows, a->pos, a->crd, b->pos, b->crd, m ? m->pos : nullptr, m ? m->crd : nullptr, g.logW,  \
            gbm, (unsigned long long *)g_sg.ticket.ptr, list, rowcount);                                   \
    } while (0)
    if (g.lds) {
        if (m) LAUNCH_SYM(true, true); else LAUNCH_SYM(true, false);
    } else {
        if (m) LAUNCH_SYM(false, true); else LAUNCH_SYM(false, false);
    }
#undef LAUNCH_SYM
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}

constexpr int SG_DENSE_MAX_BLOCKS = 64;        // the dense path serves matrices of up to 2^20 columns
// Rows with at least this many products per column block of the matrix keep their values in LDS (the span or
// the block kernel); the others add into a slab in HBM through L2 atomics.  Measured as above, ms per product
// with the span kernel in place: 128 per block 555, 64: 533, 32: 519, 16: 514, 8: 513.5, 4: 513, 1: 515.
constexpr int64_t SG_DENSE_PER_BLOCK = 8;

// Heavy rows with at least this many products per column block of the matrix stay with the block kernel, the
// others go to the span kernel (measured on A*A of an R-MAT graph of scale 20, 64 blocks, ms per product:
// 512 per block 583, 1024 572, 2048 559, 4096 557, 8192 570, every heavy row to the span kernel 604, none 613;
// with the kernels as they are now 1024 per block 437, 2048 402, 4096 386, 6144 381, 8192 382, 12288 382, 16384 389).
// COMET_HIP_SPGEMM_WIDE, a number of products per row, overrides the rule: either kernel is right for any row,
// so the tests use it to send the same rows through both.
constexpr int64_t SG_WIDE_PER_BLOCK = 6144;
static int64_t sg_wide_threshold(int nblk)
{
    const char *e = getenv("COMET_HIP_SPGEMM_WIDE");
    return e && *e ? atoll(e) : SG_WIDE_PER_BLOCK * nblk;
}

// Per-row block pointers of the right-hand operand, built once per matrix.
static int sg_plan_blocks(Csr *b)
{
    const int nblk = (int)ceil_div(b->ncols > 0 ? b->ncols : 1, SG_CB);
    if (b->sg_blkptr && b->sg_nblk == nblk)
        return COMET_HIP_OK;
    if (b->sg_blkptr) {
        COMET_HIPCHK(hipStreamSynchronize(stream()));
        COMET_HIPCHK(hipFree(b->sg_blkptr));
        (void)hipFree(b->sg_crd16);
        b->sg_blkptr = nullptr;
        b->sg_crd16 = nullptr;
    }
    static_assert(SG_CB <= 65536, "a column inside its block fits 16 bits");
    if (hipMalloc((void **)&b->sg_crd16, sizeof(uint16_t) * (size_t)(b->nnz > 0 ? b->nnz : 1)) != hipSuccess) {
        (void)hipGetLastError();        // an allocation that may fail: its error must not reach the next check
        b->sg_crd16 = nullptr;          // the kernel then reads the 32-bit columns
    } else if (b->nnz > 0) {
        spgemm_block_columns<<<dim3((unsigned)ceil_div(b->nnz, 256)), dim3(256), 0, stream()>>>(b->nnz, b->crd,
                                                                                                 b->sg_crd16);
        COMET_HIPCHK(hipGetLastError());
    }
    COMET_HIPCHK(hipMalloc((void **)&b->sg_blkptr,
                           sizeof(int64_t) * (size_t)(nblk + 1) * (size_t)(b->nrows > 0 ? b->nrows : 1)));
    b->sg_nblk = nblk;
    if (b->nrows > 0) {
        KernelTimer t("spgemm_block_pointers");
        spgemm_block_pointers<<<dim3((unsigned)ceil_div(b->nrows, 256)), dim3(256), 0, stream()>>>(
            b->nrows, b->pos, b->crd, nblk, b->sg_blkptr);
    }
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}

// ---- masked products as dot products over the mask: the host side ----
static Workspace g_dot_val, g_dot_hit, g_dot_flag;

static int dot_transposed(const Csr *x, Csr **out)
{
    Csr *m = const_cast<Csr *>(x);           // what is kept in a handle is not part of the matrix
    if (!m->transposed) {
        m->transposed = csr_transposed_copy(m);
        if (!m->transposed)
            return COMET_HIP_ERR_HIP;
    }
    *out = m->transposed;
    return COMET_HIP_OK;
}

// the transpose of the structure of x whose values say where each entry lies in x
static int dot_transposed_index(const Csr *x, Csr **out)
{
    Csr *m = const_cast<Csr *>(x);
    if (!m->transposed_index) {
        double *iota = nullptr;
        COMET_HIPCHK(hipMalloc((void **)&iota, sizeof(double) * (size_t)(m->nnz > 0 ? m->nnz : 1)));
        if (m->nnz > 0)
            fill_iota_f64<<<dim3((unsigned)ceil_div(m->nnz, 256)), dim3(256), 0, stream()>>>(m->nnz, iota);
        Csr view;
        view.nrows = m->nrows;
        view.ncols = m->ncols;
        view.nnz = m->nnz;
        view.pos = m->pos;
        view.crd = m->crd;
        view.val = iota;
        m->transposed_index = csr_transposed_copy(&view);
        const hipError_t e = hipStreamSynchronize(stream());
        (void)hipFree(iota);
        if (!m->transposed_index || e != hipSuccess)
            return set_error(COMET_HIP_ERR_HIP, "transposing the mask failed");
    }
    *out = m->transposed_index;
    return COMET_HIP_OK;
}

// whether no row of x holds a column twice (looked at once per matrix)
static int dot_no_duplicates(const Csr *x, bool *ok)
{
    Csr *m = const_cast<Csr *>(x);
    if (m->dup_state == 0) {
        COMET_CHK(g_dot_flag.ensure(sizeof(int), false));
        COMET_HIPCHK(hipMemsetAsync(g_dot_flag.ptr, 0, sizeof(int), stream()));
        if (m->nrows > 0)
            csr_find_duplicates<<<dim3((unsigned)ceil_div(m->nrows, 4)), dim3(256), 0, stream()>>>(m->nrows, m->pos, m->crd,
                                                                                                   (int *)g_dot_flag.ptr);
        int flag = 0;
        COMET_HIPCHK(hipMemcpyAsync(&flag, g_dot_flag.ptr, sizeof(int), hipMemcpyDeviceToHost, stream()));
        COMET_HIPCHK(hipStreamSynchronize(stream()));
        m->dup_state = flag ? 2 : 1;
    }
    *ok = m->dup_state == 1;
    return COMET_HIP_OK;
}

// A masked product runs as dot products when the table over k fits LDS and no list that goes into a table holds a
// column twice.  COMET_HIP_SPGEMM_NO_DOT keeps the walk over the products of every row (the tests run both).
static int dot_form_fits(const Csr *a, const Csr *b, const Csr *m, bool *fits)
{
    *fits = false;
    if (!m || a->ncols > (1ll << 20) || a->nrows >= (1ll << 31) || b->ncols >= (1ll << 31) || m->nnz >= (1ll << 52) ||
        getenv("COMET_HIP_SPGEMM_NO_DOT") != nullptr)
        return COMET_HIP_OK;
    bool ok_a = false, ok_b = false, ok_m = false;
    COMET_CHK(dot_no_duplicates(a, &ok_a));
    COMET_CHK(dot_no_duplicates(b, &ok_b));
    COMET_CHK(dot_no_duplicates(m, &ok_m));
    *fits = ok_a && ok_b && ok_m;
    return COMET_HIP_OK;
}

// pair_hit[p - Mpos[rb]] (and pair_val, with values) for every stored pair p of the mask rows [rb, re)
static int dot_pairs(const Csr *a, const Csr *b, const Csr *m, int64_t rb, int64_t re, bool values, double **pair_val,
                     uint8_t **pair_hit, int reduce_op, int mult_op)
{
    const bool semi = reduce_op != COMET_SR_PLUS || mult_op != COMET_OP_TIMES;
    Csr *bt = nullptr, *mt = nullptr;
    COMET_CHK(dot_transposed(b, &bt));
    COMET_CHK(dot_transposed_index(m, &mt));
    int64_t ends[2] = {0, 0};
    COMET_HIPCHK(hipMemcpyAsync(&ends[0], m->pos + rb, sizeof(int64_t), hipMemcpyDeviceToHost, stream()));
    COMET_HIPCHK(hipMemcpyAsync(&ends[1], m->pos + re, sizeof(int64_t), hipMemcpyDeviceToHost, stream()));
    COMET_HIPCHK(hipStreamSynchronize(stream()));
    const int64_t out0 = ends[0], npairs = ends[1] - ends[0];
    COMET_CHK(g_dot_hit.ensure((size_t)(npairs > 0 ? npairs : 1), false));
    COMET_CHK(g_dot_val.ensure(sizeof(double) * (size_t)(npairs > 0 ? npairs : 1), false));
    *pair_hit = (uint8_t *)g_dot_hit.ptr;
    *pair_val = (double *)g_dot_val.ptr;
    if (npairs == 0)
        return COMET_HIP_OK;
    COMET_HIPCHK(hipMemsetAsync(*pair_hit, 0, (size_t)npairs, stream()));
    if (values)
        COMET_HIPCHK(hipMemsetAsync(*pair_val, 0, sizeof(double) * (size_t)npairs, stream()));
    int words = (int)ceil_div(a->ncols > 0 ? a->ncols : 1, 32);
    words = (int)ceil_div(words, DT_WPT) * DT_WPT;
    const size_t lds = dot_lds_bytes(words);
    if (dot_table_words(words) % 2 != 0 || words % DT_WPT != 0)        // the wavefronts' fp64 sums follow the table
        return set_error(COMET_HIP_ERR_SIZE, "dot-product table of %d words leaves its sums misaligned", words);
    const dim3 grid((unsigned)(num_cus() > 0 ? num_cus() : 256)), block(SG_T);
    const int64_t everywhere = 1ll << 62;
    for (int half = 0; half < 2; ++half) {
        // the row's half: tables of the rows of A, the columns of B streamed; the column's half the other way round
        const Csr *T = half == 0 ? a : bt, *P = half == 0 ? m : mt, *L = half == 0 ? bt : a;
        const int64_t first = half == 0 ? rb : 0, last = half == 0 ? re : mt->nrows;
        RowList list;        // the rows that have pairs of this half, by the entries these stream
        SgPairFilter mine;
        mine.towner = T;
        mine.strict = half;
        mine.xlo = half == 0 ? 0 : rb;
        mine.xhi = half == 0 ? everywhere : re;
        COMET_CHK(sg_row_list(P, L, first, last, SG_NO_DENSE, SG_NO_DENSE, &list, nullptr, 0, mine));
        COMET_CHK(sg_reset_ticket());
        KernelTimer t(values ? (half == 0 ? "spgemm_numeric_dot_rows" : "spgemm_numeric_dot_columns")
                             : (half == 0 ? "spgemm_symbolic_dot_rows" : "spgemm_symbolic_dot_columns"));
#define LAUNCH_DOT(V, S)                                                                                   \
    do {                                                                                                   \
        COMET_CHK(sg_allow_lds(spgemm_dot_kernel<V, S>, lds));                                             \
        spgemm_dot_kernel<V, S><<<grid, block, lds, stream()>>>(                                           \
            first, T->pos, T->crd, T->val, P->pos, P->crd, L->pos, L->crd, L->val,                         \
            half == 0 ? nullptr : mt->val, out0, half, half == 0 ? 0 : rb, half == 0 ? everywhere : re,    \
            words, (unsigned long long *)g_sg.ticket.ptr, list, *pair_val, *pair_hit, reduce_op, mult_op,  \
            half);                                                                                         \
    } while (0)
        if (!values)
            LAUNCH_DOT(false, false);
        else if (semi)
            LAUNCH_DOT(true, true);
        else
            LAUNCH_DOT(true, false);
#undef LAUNCH_DOT
        COMET_HIPCHK(hipGetLastError());
    }
    return COMET_HIP_OK;
}

static int numeric_rows(const Csr *a, Csr *b, const Csr *m, const int64_t *Cpos, int64_t rb, int64_t re,
                        int32_t *Ccrd, double *Cval, int reduce_op, int mult_op)
{
    if (reduce_op < 0 || reduce_op > COMET_SR_ANY || mult_op < 0 || mult_op > COMET_OP_DIV)
        return set_error(COMET_HIP_ERR_ARG, "unknown semiring (reduce %d, mult %d)", reduce_op, mult_op);
    const bool semi = reduce_op != COMET_SR_PLUS || mult_op != COMET_OP_TIMES;
    if (m && reduce_op != COMET_SR_ANY && re > rb) {
        bool dots = false;
        COMET_CHK(dot_form_fits(a, b, m, &dots));
        if (dots) {
            double *pair_val = nullptr;
            uint8_t *pair_hit = nullptr;
            COMET_CHK(dot_pairs(a, b, m, rb, re, true, &pair_val, &pair_hit, reduce_op, mult_op));
            KernelTimer t("spgemm_numeric_dot_compact");
            spgemm_dot_compact<<<dim3((unsigned)ceil_div(re - rb, 4)), dim3(256), 0, stream()>>>(
                rb, re, m->pos, m->crd, pair_val, pair_hit, Cpos, Ccrd, Cval);
            COMET_HIPCHK(hipGetLastError());
            return COMET_HIP_OK;
        }
    }
    SgGeom g;
    COMET_CHK(sg_geometry(b->ncols, &g));
    COMET_CHK(sg_reset_ticket());
    // rows with many products go to the LDS-accumulator kernel (unmasked products only)
    const int nblk = (int)ceil_div(b->ncols > 0 ? b->ncols : 1, SG_CB);
    // (the `any` semiring keeps a product's place in B in 32 bits of its accumulator)
    const bool lds_rows = nblk <= SG_DENSE_MAX_BLOCKS && (reduce_op != COMET_SR_ANY || b->nnz < (1ll << 32));
    const bool dense = !m && lds_rows;
    // masked: the rows whose mask row does not fit the slab kernel's hash table take the one-block kernel
    const bool mdense = m && lds_rows && g.lds && getenv("COMET_HIP_SPGEMM_NO_MASKED_DENSE") == nullptr;
    const int64_t dense_threshold = dense ? SG_DENSE_PER_BLOCK * nblk : SG_NO_DENSE;
    if (dense || mdense)
        COMET_CHK(sg_plan_blocks(b));
    RowList list;
    const int64_t wide = sg_wide_threshold(nblk) > dense_threshold ? sg_wide_threshold(nblk) : dense_threshold;
    if (mdense)         // those rows sort in front (sg_row_keys): bounds[0] = bounds[2] = their number
        COMET_CHK(sg_row_list(a, b, rb, re, 1ll << 61, 1ll << 61, &list, m, SG_HASH_FILL));
    else
        COMET_CHK(sg_row_list(a, b, rb, re, dense_threshold, dense ? wide : SG_NO_DENSE, &list));
    uint32_t *gbm = nullptr, *gmask = nullptr;
    if (!g.lds || m) {          // the output row's bitmap is in HBM when LDS holds the mask row instead
        COMET_CHK(g_sg.gbm.ensure(sizeof(uint32_t) * g.bm_words * (size_t)g.groups, true));
        gbm = (uint32_t *)g_sg.gbm.ptr;
    }
    if (m && !g.lds) {
        COMET_CHK(g_sg.gmask.ensure(sizeof(uint32_t) * g.bm_words * (size_t)g.groups, true));
        gmask = (uint32_t *)g_sg.gmask.ptr;
    }
    COMET_CHK(g_sg.slabs.ensure(sizeof(double) * (size_t)(b->ncols > 0 ? b->ncols : 1) * (size_t)g.groups, true));
    const dim3 grid((unsigned)g.groups), block(SG_T);
    // a masked product keeps either the mask row's bitmap or its hash table in LDS, whichever the row needs
    const size_t num_lds = m && g.lds && g.lds_bytes < SG_HASH_LDS ? SG_HASH_LDS : g.lds_bytes;
#define LAUNCH_NUM(L, M, S)                                                                                \
    do {                                                                                                   \
        COMET_CHK(sg_allow_lds(spgemm_numeric_kernel<L, M, S>, num_lds));                                  \
        KernelTimer t(S ? "spgemm_numeric_semiring" : M ? "spgemm_numeric_masked" : "spgemm_numeric");    \
        spgemm_numeric_kernel<L, M, S><<<grid, block, num_lds, stream()>>>(                                \
            rb, re, b->ncols, a->pos, a->crd, a->val, b->pos, b->crd, b->val, m ? m->pos : nullptr,        \
            m ? m->crd : nullptr, g.logW, gbm, gmask, (double *)g_sg.slabs.ptr,                            \
            (unsigned long long *)g_sg.ticket.ptr, list, 1, reduce_op, mult_op, Cpos, Ccrd, Cval);         \
    } while (0)
#define LAUNCH_NUM_S(L, M)                                                                                 \
    do {                                                                                                   \
        if (semi) LAUNCH_NUM(L, M, true); else LAUNCH_NUM(L, M, false);                                    \
    } while (0)
    if (g.lds) {
        if (m) LAUNCH_NUM_S(true, true); else LAUNCH_NUM_S(true, false);
    } else {
        if (m) LAUNCH_NUM_S(false, true); else LAUNCH_NUM_S(false, false);
    }
#undef LAUNCH_NUM_S
#undef LAUNCH_NUM
    COMET_HIPCHK(hipGetLastError());
    // the rows of the one-block kernel block by block (COMET_HIP_SPGEMM_ROW_MAJOR keeps them row by row; the
    // tests run both)
    const bool by_blocks = dense && a->nnz < (1ll << 30) && getenv("COMET_HIP_SPGEMM_ROW_MAJOR") == nullptr;
    bool ran_blocks = false;
    if (by_blocks) {
        int64_t nd = 0;
        COMET_HIPCHK(hipMemcpyAsync(&nd, list.bounds + 2, sizeof(int64_t), hipMemcpyDeviceToHost, stream()));
        COMET_HIPCHK(hipStreamSynchronize(stream()));
        if (nd > 0) {
            ran_blocks = true;
            COMET_CHK(g_sg.dense_rows.ensure(sizeof(DenseRow) * (size_t)nd, false));
            COMET_CHK(g_sg.dense_before.ensure(sizeof(int32_t) * (size_t)nd * (size_t)nblk, false));
            COMET_CHK(g_sg.gave_up.ensure(sizeof(int), true));
            // cleared before every launch that can set it: a call that fails between the launch and the read
            // below must not leave it set for the next product
            COMET_HIPCHK(hipMemsetAsync(g_sg.gave_up.ptr, 0, sizeof(int), stream()));
            COMET_CHK(sg_reset_ticket());
            int patience = DB_PATIENCE;
            if (const char *e = getenv("COMET_HIP_SPGEMM_PATIENCE"))
                patience = atoi(e);
            KernelTimer t("spgemm_numeric_dense_blocks");
            const dim3 cus((unsigned)(num_cus() > 0 ? num_cus() : 256));
            spgemm_dense_rows<<<dim3((unsigned)ceil_div(nd * nblk, 256)), dim3(256), 0, stream()>>>(
                rb, list, nd, nblk, a->pos, Cpos, (DenseRow *)g_sg.dense_rows.ptr, (int32_t *)g_sg.dense_before.ptr);
#define LAUNCH_BLOCKS_C(S, COL, CRD)                                                                       \
    do {                                                                                                   \
        COMET_CHK(sg_allow_lds(spgemm_numeric_dense_blocks_kernel<S, COL>, SG_DENSE_LDS));                 \
        spgemm_numeric_dense_blocks_kernel<S, COL><<<cus, block, SG_DENSE_LDS, stream()>>>(                \
            (const DenseRow *)g_sg.dense_rows.ptr, nd, a->crd, a->val, CRD, b->val, b->sg_blkptr, nblk,    \
            (unsigned long long *)g_sg.ticket.ptr, (int32_t *)g_sg.dense_before.ptr, patience,             \
            (int *)g_sg.gave_up.ptr, Ccrd, Cval, reduce_op, mult_op);                                      \
    } while (0)
#define LAUNCH_BLOCKS(S)                                                                                   \
    do {                                                                                                   \
        if (b->sg_crd16 && getenv("COMET_HIP_SPGEMM_WIDE_COLUMNS") == nullptr)                             \
            LAUNCH_BLOCKS_C(S, uint16_t, b->sg_crd16);                                                     \
        else                                                                                               \
            LAUNCH_BLOCKS_C(S, int32_t, b->crd);                                                           \
    } while (0)
            if (semi) LAUNCH_BLOCKS(true); else LAUNCH_BLOCKS(false);
#undef LAUNCH_BLOCKS_C
#undef LAUNCH_BLOCKS
            COMET_HIPCHK(hipGetLastError());
        }
    }
    if ((dense && !by_blocks) || mdense) {
        COMET_CHK(sg_reset_ticket());
        KernelTimer t(mdense ? "spgemm_numeric_dense_masked" : "spgemm_numeric_dense");
        const dim3 cus((unsigned)(num_cus() > 0 ? num_cus() : 256));
#define LAUNCH_DENSE_C(S, M, COL, CRD)                                                                     \
    do {                                                                                                   \
        COMET_CHK(sg_allow_lds(spgemm_numeric_dense_kernel<S, M, COL>, SG_DENSE_LDS));                     \
        spgemm_numeric_dense_kernel<S, M, COL><<<cus, block, SG_DENSE_LDS, stream()>>>(                    \
            rb, re, a->pos, a->crd, a->val, CRD, b->val, m ? m->pos : nullptr, m ? m->crd : nullptr,       \
            b->sg_blkptr, nblk, (unsigned long long *)g_sg.ticket.ptr, list, Cpos, Ccrd, Cval, reduce_op,  \
            mult_op);                                                                                      \
    } while (0)
#define LAUNCH_DENSE(S, M)                                                                                 \
    do {                                                                                                   \
        if (b->sg_crd16 && getenv("COMET_HIP_SPGEMM_WIDE_COLUMNS") == nullptr)                             \
            LAUNCH_DENSE_C(S, M, uint16_t, b->sg_crd16);                                                   \
        else                                                                                               \
            LAUNCH_DENSE_C(S, M, int32_t, b->crd);                                                         \
    } while (0)
        if (mdense) {
            if (semi) LAUNCH_DENSE(true, true); else LAUNCH_DENSE(false, true);
        } else {
            if (semi) LAUNCH_DENSE(true, false); else LAUNCH_DENSE(false, false);
        }
#undef LAUNCH_DENSE_C
#undef LAUNCH_DENSE
        COMET_HIPCHK(hipGetLastError());
    }
    if (dense) {
        COMET_CHK(sg_reset_ticket());
        KernelTimer t("spgemm_numeric_span");
        const dim3 cus((unsigned)(num_cus() > 0 ? num_cus() : 256));
        if (semi) {
            COMET_CHK(sg_allow_lds(spgemm_numeric_span_kernel<true>, SG_SPAN_LDS));
            spgemm_numeric_span_kernel<true><<<cus, block, SG_SPAN_LDS, stream()>>>(
                rb, re, a->pos, a->crd, a->val, b->crd, b->val, b->sg_blkptr, nblk,
                (unsigned long long *)g_sg.ticket.ptr, list, Cpos, Ccrd, Cval, reduce_op, mult_op);
        } else {
            COMET_CHK(sg_allow_lds(spgemm_numeric_span_kernel<false>, SG_SPAN_LDS));
            spgemm_numeric_span_kernel<false><<<cus, block, SG_SPAN_LDS, stream()>>>(
                rb, re, a->pos, a->crd, a->val, b->crd, b->val, b->sg_blkptr, nblk,
                (unsigned long long *)g_sg.ticket.ptr, list, Cpos, Ccrd, Cval, reduce_op, mult_op);
        }
        COMET_HIPCHK(hipGetLastError());
    }
    if (ran_blocks) {           // did a workgroup stop waiting for the block before its own
        int gave_up = 0;
        COMET_HIPCHK(hipMemcpyAsync(&gave_up, g_sg.gave_up.ptr, sizeof(int), hipMemcpyDeviceToHost, stream()));
        COMET_HIPCHK(hipStreamSynchronize(stream()));
        if (gave_up) {
            COMET_HIPCHK(hipMemsetAsync(g_sg.gave_up.ptr, 0, sizeof(int), stream()));
            return set_error(COMET_HIP_ERR_HIP, "spgemm numeric: a column block's place in its row never arrived");
        }
    }
    return COMET_HIP_OK;
}

}  // namespace comet

using namespace comet;

extern "C" int comet_hip_spgemm_csr_symbolic(int64_t ah, int64_t bh, int64_t mh, int64_t pos_dptr, int64_t *nnz_out)
{
    COMET_CHK(ensure_init());
    Csr *a = csr_from_handle(ah), *b = csr_from_handle(bh), *m = mh ? csr_from_handle(mh) : nullptr;
    if (!a || !b || (mh && !m))
        return COMET_HIP_ERR_HANDLE;
    if (!pos_dptr)
        return set_error(COMET_HIP_ERR_ARG, "null pos passed to comet_hip_spgemm_csr_symbolic");
    COMET_CHK(check_product_shapes(a, b, m, "spgemm symbolic"));
    int64_t *pos = (int64_t *)pos_dptr;
    if (a->nrows > 0) {
        COMET_CHK(g_sg.rowcount.ensure(sizeof(int64_t) * (size_t)a->nrows, false));
        COMET_CHK(symbolic_counts(a, b, m, (int64_t *)g_sg.rowcount.ptr));
    }
    COMET_CHK(exclusive_scan_i64((const int64_t *)g_sg.rowcount.ptr, a->nrows, pos));
    if (nnz_out) {
        COMET_HIPCHK(hipMemcpyAsync(nnz_out, pos + a->nrows, sizeof(int64_t), hipMemcpyDeviceToHost, stream()));
        COMET_HIPCHK(hipStreamSynchronize(stream()));
    }
    return COMET_HIP_OK;
}

extern "C" int comet_hip_spgemm_csr_numeric(int64_t ah, int64_t bh, int64_t mh, int64_t pos_dptr, int64_t row_begin,
                                            int64_t row_end, int64_t crd_dptr, int64_t val_dptr)
{
    return comet_hip_spgemm_csr_numeric_semiring(ah, bh, mh, pos_dptr, row_begin, row_end, crd_dptr, val_dptr,
                                                 COMET_SR_PLUS, COMET_OP_TIMES);
}

extern "C" int comet_hip_spgemm_csr_numeric_semiring(int64_t ah, int64_t bh, int64_t mh, int64_t pos_dptr,
                                                     int64_t row_begin, int64_t row_end, int64_t crd_dptr,
                                                     int64_t val_dptr, int reduce_op, int mult_op)
{
    COMET_CHK(ensure_init());
    Csr *a = csr_from_handle(ah), *b = csr_from_handle(bh), *m = mh ? csr_from_handle(mh) : nullptr;
    if (!a || !b || (mh && !m))
        return COMET_HIP_ERR_HANDLE;
    COMET_CHK(check_product_shapes(a, b, m, "spgemm numeric"));
    if (row_begin < 0 || row_end < row_begin || row_end > a->nrows)
        return set_error(COMET_HIP_ERR_ARG, "row range [%lld,%lld) outside [0,%lld]", (long long)row_begin,
                         (long long)row_end, (long long)a->nrows);
    if (!pos_dptr || !crd_dptr || !val_dptr)
        return set_error(COMET_HIP_ERR_ARG, "null output array passed to comet_hip_spgemm_csr_numeric");
    if (row_begin == row_end)
        return COMET_HIP_OK;
    return numeric_rows(a, b, m, (const int64_t *)pos_dptr, row_begin, row_end, (int32_t *)crd_dptr,
                        (double *)val_dptr, reduce_op, mult_op);
}

extern "C" int64_t comet_hip_spgemm_csr(int64_t ah, int64_t bh, int64_t mh)
{
    return comet_hip_spgemm_csr_semiring(ah, bh, mh, COMET_SR_PLUS, COMET_OP_TIMES);
}

// C<M> = A*B in one pass over the pairs of the mask: their values and which of them met a product come out of
// the same walk, so the row pointers need no symbolic phase of their own.  *done says whether this form applied.
static int64_t masked_product_one_pass(const Csr *a, const Csr *b, const Csr *m, int reduce_op, int mult_op, bool *done)
{
    *done = false;
    bool dots = false;
    if (dot_form_fits(a, b, m, &dots) != COMET_HIP_OK)
        return 0;
    if (!dots || a->nrows == 0)
        return 0;
    *done = true;
    double *pair_val = nullptr;
    uint8_t *pair_hit = nullptr;
    if (dot_pairs(a, b, m, 0, a->nrows, true, &pair_val, &pair_hit, reduce_op, mult_op) != COMET_HIP_OK ||
        g_sg.rowcount.ensure(sizeof(int64_t) * (size_t)a->nrows, false) != COMET_HIP_OK)
        return 0;
    Csr *c = new Csr();
    c->nrows = a->nrows;
    c->ncols = b->ncols;
    c->owns = true;
    const auto fail = [&](const char *what) -> int64_t {
        if (what)
            set_error(COMET_HIP_ERR_HIP, "%s", what);
        csr_release(c);
        return 0;
    };
    if (hipMalloc((void **)&c->pos, sizeof(int64_t) * (size_t)(a->nrows + 1)) != hipSuccess)
        return fail("row pointer allocation failed");
    {
        KernelTimer t("spgemm_symbolic_dot_count");
        spgemm_dot_count<<<dim3((unsigned)ceil_div(a->nrows, 4)), dim3(256), 0, stream()>>>(
            0, a->nrows, m->pos, pair_hit, (int64_t *)g_sg.rowcount.ptr);
    }
    if (exclusive_scan_i64((const int64_t *)g_sg.rowcount.ptr, a->nrows, c->pos) != COMET_HIP_OK)
        return fail(nullptr);
    if (hipMemcpyAsync(&c->nnz, c->pos + a->nrows, sizeof(int64_t), hipMemcpyDeviceToHost, stream()) != hipSuccess ||
        hipStreamSynchronize(stream()) != hipSuccess)
        return fail("reading the size of the product failed");
    if (hipMalloc((void **)&c->crd, sizeof(int32_t) * (size_t)(c->nnz > 0 ? c->nnz : 1)) != hipSuccess ||
        hipMalloc((void **)&c->val, sizeof(double) * (size_t)(c->nnz > 0 ? c->nnz : 1)) != hipSuccess)
        return fail("output allocation failed");
    {
        KernelTimer t("spgemm_numeric_dot_compact");
        spgemm_dot_compact<<<dim3((unsigned)ceil_div(a->nrows, 4)), dim3(256), 0, stream()>>>(
            0, a->nrows, m->pos, m->crd, pair_val, pair_hit, c->pos, c->crd, c->val);
    }
    if (hipGetLastError() != hipSuccess)
        return fail("launching the compaction failed");
    return csr_register(c);
}

extern "C" int64_t comet_hip_spgemm_csr_semiring(int64_t ah, int64_t bh, int64_t mh, int reduce_op, int mult_op)
{
    if (ensure_init() != COMET_HIP_OK)
        return 0;
    Csr *a = csr_from_handle(ah), *b = csr_from_handle(bh), *m = mh ? csr_from_handle(mh) : nullptr;
    if (!a || !b || (mh && !m))
        return 0;
    if (check_product_shapes(a, b, m, "spgemm") != COMET_HIP_OK)
        return 0;
    if (m && reduce_op >= 0 && reduce_op < COMET_SR_ANY && mult_op >= 0 && mult_op <= COMET_OP_DIV) {
        bool done = false;
        const int64_t h = masked_product_one_pass(a, b, m, reduce_op, mult_op, &done);
        if (done)
            return h;
    }
    int64_t *pos = nullptr;
    if (hipMalloc((void **)&pos, sizeof(int64_t) * (size_t)(a->nrows + 1)) != hipSuccess) {
        set_error(COMET_HIP_ERR_HIP, "row pointer allocation failed");
        return 0;
    }
    int64_t nnz = 0;
    if (comet_hip_spgemm_csr_symbolic(ah, bh, mh, (int64_t)pos, &nnz) != COMET_HIP_OK) {
        (void)hipFree(pos);
        return 0;
    }
    Csr *c = new Csr();
    c->nrows = a->nrows;
    c->ncols = b->ncols;
    c->nnz = nnz;
    c->pos = pos;
    c->owns = true;
    if (hipMalloc((void **)&c->crd, sizeof(int32_t) * (size_t)(nnz > 0 ? nnz : 1)) != hipSuccess ||
        hipMalloc((void **)&c->val, sizeof(double) * (size_t)(nnz > 0 ? nnz : 1)) != hipSuccess) {
        set_error(COMET_HIP_ERR_HIP, "output allocation of %lld entries failed", (long long)nnz);
        (void)hipFree(c->crd);
        (void)hipFree(pos);
        delete c;
        return 0;
    }
    if (nnz > 0 && numeric_rows(a, b, m, pos, 0, a->nrows, c->crd, c->val, reduce_op, mult_op) != COMET_HIP_OK) {
        (void)hipFree(c->crd);
        (void)hipFree(c->val);
        (void)hipFree(pos);
        delete c;
        return 0;
    }
    return csr_register(c);
}

static int csr_is_iso(const Csr *x, bool *iso)
{
    Csr *m = const_cast<Csr *>(x);
    if (m->iso_state == 0) {
        int flag = 1;
        if (m->nnz > 0) {
            COMET_CHK(g_dot_flag.ensure(sizeof(int), false));
            COMET_HIPCHK(hipMemsetAsync(g_dot_flag.ptr, 0, sizeof(int), stream()));
            csr_values_differ<<<dim3((unsigned)ceil_div(m->nnz, 256)), dim3(256), 0, stream()>>>(m->nnz, m->val,
                                                                                                (int *)g_dot_flag.ptr);
            COMET_HIPCHK(hipGetLastError());
            COMET_HIPCHK(hipMemcpyAsync(&flag, g_dot_flag.ptr, sizeof(int), hipMemcpyDeviceToHost, stream()));
            COMET_HIPCHK(hipMemcpyAsync(&m->iso_value, m->val, sizeof(double), hipMemcpyDeviceToHost, stream()));
            COMET_HIPCHK(hipStreamSynchronize(stream()));
        }
        m->iso_state = flag ? 2 : 1;
    }
    *iso = m->iso_state == 1;
    return COMET_HIP_OK;
}

extern "C" int comet_hip_spgemm_masked_sum(int64_t ah, int64_t bh, int64_t mh, double *out)
{
    COMET_CHK(ensure_init());
    Csr *a = csr_from_handle(ah), *b = csr_from_handle(bh), *m = csr_from_handle(mh);
    if (!a || !b || !m)
        return COMET_HIP_ERR_HANDLE;
    if (!out)
        return set_error(COMET_HIP_ERR_ARG, "null result pointer");
    COMET_CHK(check_product_shapes(a, b, m, "masked sum"));
    if (a->nrows == 0) {
        *out = 0.0;
        return COMET_HIP_OK;
    }
    SgGeom g;
    COMET_CHK(sg_geometry(b->ncols, &g));
    COMET_CHK(sg_reset_ticket());
    COMET_CHK(g_sg.rowcount.ensure(sizeof(double) * (size_t)a->nrows, false));
    uint32_t *gbm = nullptr;
    if (!g.lds) {
        COMET_CHK(g_sg.gbm.ensure(sizeof(uint32_t) * g.bm_words * (size_t)g.groups, true));
        gbm = (uint32_t *)g_sg.gbm.ptr;
    }
    double *rowsum = (double *)g_sg.rowcount.ptr;
    RowList list;
    // rows whose mask row is too long for the wavefront kernel's table sort to the front, whatever their products:
    // the workgroup kernel, which starts there, looks a column up in one LDS read; the wavefront kernel would
    // bisect the mask row in memory for every product
    bool iso = false;
    if (g.lds)
        COMET_CHK(csr_is_iso(b, &iso));
    COMET_CHK(sg_row_list(a, b, 0, a->nrows, SG_NO_DENSE, SG_NO_DENSE, &list, m, iso ? SI_MASK_MAX : SM_MASK_MAX));
    COMET_HIPCHK(hipMemsetAsync(rowsum, 0, sizeof(double) * (size_t)a->nrows, stream()));
    const dim3 grid((unsigned)g.groups), block(SG_T);
    // Two kernels side by side, the second on the auxiliary stream: a workgroup per row from the heavy end of
    // the list, a wavefront per row from the light end, until they meet.  A row of a thousand products costs
    // the first kernel more in barriers than in products; a row of a million would keep one wavefront of the
    // second busy for a millisecond.  Triangle count of the scale-20 R-MAT graph: 29.2 ms with the first
    // kernel alone, 22.1 ms one after the other with a fixed split at 65536 products, 17.6 ms side by side with
    // the best fixed split (49152 products), 18.9 ms with the two ends meeting by themselves (the difference is
    // the last wavefront-rows near the meeting point; looking at the ticket word before drawing from it, to keep
    // the wavefronts away from those rows, or drawing 16 rows at a time, costs more on that one word than it saves).
    // COMET_HIP_MASKED_SUM_ONLY=workgroup|wavefront launches one of the two kernels only, which then takes every
    // row: the tests send each class of rows through both
    const char *only = getenv("COMET_HIP_MASKED_SUM_ONLY");
    const bool run_wg = !only || strcmp(only, "wavefront") != 0, run_wave = !only || strcmp(only, "workgroup") != 0;
    COMET_CHK(aux_fork());
    if (!run_wg) {
    } else if (iso) {
        const int nwords = (int)ceil_div(b->ncols, 32);
        COMET_CHK(sg_allow_lds(spgemm_masked_sum_iso_kernel, sizeof(uint32_t) * (size_t)nwords));
        KernelTimer t("spgemm_masked_sum");
        // Not a workgroup for every CU: beside one, a CU's registers hold a single wavefront of the other kernel per
        // SIMD, and the half million light rows that kernel takes each wait on memory four times in a row.  The
        // CUs left free hold sixteen of its wavefronts (triangle count of the scale-20 graph: 5.2 ms with a
        // workgroup on every CU, 4.76 ms on 208 to 224 of 256, 5.7 ms on 192).
        // That single wavefront per SIMD is there only as long as this kernel keeps to 96 vector registers (four
        // wavefronts of 96 and one of the other kernel's 112 make 496 of a SIMD's 512): with 97 it is allotted 104,
        // the other kernel is left with the free CUs alone and the count takes 6.6 ms.
        const dim3 igrid(g.groups == num_cus() ? (unsigned)(g.groups - 3 * (g.groups / 16)) : (unsigned)g.groups);
        spgemm_masked_sum_iso_kernel<<<igrid, block, sizeof(uint32_t) * (size_t)nwords, stream()>>>(
            a->pos, a->crd, a->val, b->pos, b->crd, b->iso_value, m->pos, m->crd, nwords,
            (unsigned long long *)g_sg.ticket.ptr, list, rowsum);
    } else if (g.lds) {
        COMET_CHK(sg_allow_lds(spgemm_masked_sum_kernel<true>, g.lds_bytes));
        KernelTimer t("spgemm_masked_sum");
        spgemm_masked_sum_kernel<true><<<grid, block, g.lds_bytes, stream()>>>(
            a->nrows, a->pos, a->crd, a->val, b->pos, b->crd, b->val, m->pos, m->crd, g.logW, gbm,
            (unsigned long long *)g_sg.ticket.ptr, list, rowsum);
    } else {
        KernelTimer t("spgemm_masked_sum");
        spgemm_masked_sum_kernel<false><<<grid, block, 0, stream()>>>(
            a->nrows, a->pos, a->crd, a->val, b->pos, b->crd, b->val, m->pos, m->crd, g.logW, gbm,
            (unsigned long long *)g_sg.ticket.ptr, list, rowsum);
    }
    if (run_wave && iso) {
        KernelTimer t("spgemm_masked_sum_small", aux_stream());
        spgemm_masked_sum_small_iso_kernel<<<dim3((unsigned)(num_cus() * 8)), dim3(SM_WAVES * 64), 0, aux_stream()>>>(
            a->pos, a->crd, a->val, b->pos, b->crd, b->iso_value, m->pos, m->crd,
            (unsigned long long *)g_sg.ticket.ptr, list, rowsum);
    } else if (run_wave) {   // eight workgroups of four wavefronts per CU: four fit beside the kernel above, the rest follow it
        KernelTimer t("spgemm_masked_sum_small", aux_stream());
        spgemm_masked_sum_small_kernel<<<dim3((unsigned)(num_cus() * 8)), dim3(SM_WAVES * 64), 0, aux_stream()>>>(
            a->pos, a->crd, a->val, b->pos, b->crd, b->val, m->pos, m->crd,
            (unsigned long long *)g_sg.ticket.ptr, list, rowsum);
    }
    COMET_HIPCHK(hipGetLastError());
    COMET_CHK(aux_join());
    return reduce_sum_device(rowsum, a->nrows, out);
}

extern "C" int64_t comet_hip_eltwise_mult_csr(int64_t ah, int64_t bh)
{
    if (ensure_init() != COMET_HIP_OK)
        return 0;
    Csr *a = csr_from_handle(ah), *b = csr_from_handle(bh);
    if (!a || !b)
        return 0;
    if (a->nrows != b->nrows || a->ncols != b->ncols) {
        set_error(COMET_HIP_ERR_ARG, "element-wise product of %lld x %lld and %lld x %lld", (long long)a->nrows,
                  (long long)a->ncols, (long long)b->nrows, (long long)b->ncols);
        return 0;
    }
    const int64_t n = a->nrows;
    int64_t *pos = nullptr;
    if (hipMalloc((void **)&pos, sizeof(int64_t) * (size_t)(n + 1)) != hipSuccess) {
        set_error(COMET_HIP_ERR_HIP, "row pointer allocation failed");
        return 0;
    }
    auto fail = [&](Csr *c) -> int64_t {
        if (c) {
            (void)hipFree(c->crd);
            (void)hipFree(c->val);
            delete c;
        }
        (void)hipFree(pos);
        return 0;
    };
    if (g_sg.rowcount.ensure(sizeof(int64_t) * (size_t)(n > 0 ? n : 1), false) != COMET_HIP_OK)
        return fail(nullptr);
    int64_t *rowcount = (int64_t *)g_sg.rowcount.ptr;
    const dim3 grid((unsigned)ceil_div(n > 0 ? n : 1, 256)), block(256);
    if (n > 0) {
        KernelTimer t("eltwise_mult_count");
        eltwise_mult_kernel<false><<<grid, block, 0, stream()>>>(n, a->pos, a->crd, a->val, b->pos, b->crd, b->val,
                                                                 rowcount, nullptr, nullptr, nullptr);
    }
    if (exclusive_scan_i64(rowcount, n, pos) != COMET_HIP_OK)
        return fail(nullptr);
    int64_t nnz = 0;
    if (hipMemcpyAsync(&nnz, pos + n, sizeof(int64_t), hipMemcpyDeviceToHost, stream()) != hipSuccess ||
        hipStreamSynchronize(stream()) != hipSuccess) {
        set_error(COMET_HIP_ERR_HIP, "reading nnz failed");
        return fail(nullptr);
    }
    Csr *c = new Csr();
    c->nrows = n;
    c->ncols = a->ncols;
    c->nnz = nnz;
    c->pos = pos;
    c->owns = true;
    if (hipMalloc((void **)&c->crd, sizeof(int32_t) * (size_t)(nnz > 0 ? nnz : 1)) != hipSuccess ||
        hipMalloc((void **)&c->val, sizeof(double) * (size_t)(nnz > 0 ? nnz : 1)) != hipSuccess) {
        set_error(COMET_HIP_ERR_HIP, "output allocation failed");
        return fail(c);
    }
    if (n > 0 && nnz > 0) {
        KernelTimer t("eltwise_mult_fill");
        eltwise_mult_kernel<true><<<grid, block, 0, stream()>>>(n, a->pos, a->crd, a->val, b->pos, b->crd, b->val,
                                                                nullptr, pos, c->crd, c->val);
    }
    if (hipGetLastError() != hipSuccess) {
        set_error(COMET_HIP_ERR_HIP, "element-wise kernel launch failed");
        return fail(c);
    }
    return csr_register(c);
}

extern "C" int64_t comet_hip_eltwise_csr_dense_csr(int64_t ah, int64_t d_dptr, int64_t ldd, int op)
{
    if (ensure_init() != COMET_HIP_OK)
        return 0;
    Csr *a = csr_from_handle(ah);
    if (!a)
        return 0;
    if (ldd < a->ncols || (a->nnz > 0 && !d_dptr) || op < 0 || op > COMET_OP_DIV) {
        set_error(COMET_HIP_ERR_ARG, "bad dense operand or operator passed to comet_hip_eltwise_csr_dense_csr");
        return 0;
    }
    Csr *c = new Csr();
    if (csr_alloc(c, a->nrows, a->ncols, a->nnz) != COMET_HIP_OK) {
        delete c;
        return 0;
    }
    bool ok = hipMemcpyAsync(c->pos, a->pos, sizeof(int64_t) * (size_t)(a->nrows + 1), hipMemcpyDeviceToDevice,
                             stream()) == hipSuccess;
    if (ok && a->nnz > 0) {
        ok = hipMemcpyAsync(c->crd, a->crd, sizeof(int32_t) * (size_t)a->nnz, hipMemcpyDeviceToDevice, stream()) ==
             hipSuccess;
        KernelTimer t("eltwise_mult_dense");
        eltwise_mult_dense_kernel<false><<<dim3((unsigned)ceil_div(a->nrows * 16, 256)), dim3(256), 0, stream()>>>(
            a->nrows, a->pos, a->crd, a->val, (const double *)d_dptr, ldd, c->val, 0, op);
    }
    if (!ok || hipGetLastError() != hipSuccess) {
        set_error(COMET_HIP_ERR_HIP, "CSR .* Dense failed");
        csr_release(c);
        return 0;
    }
    return csr_register(c);
}

extern "C" int comet_hip_eltwise_csr_dense_dense(int64_t ah, int64_t d_dptr, int64_t ldd, int64_t c_dptr,
                                                 int64_t ldc, int op)
{
    COMET_CHK(ensure_init());
    Csr *a = csr_from_handle(ah);
    if (!a)
        return COMET_HIP_ERR_HANDLE;
    if (ldd < a->ncols || ldc < a->ncols || (a->nnz > 0 && (!d_dptr || !c_dptr)) || op < 0 || op > COMET_OP_DIV)
        return set_error(COMET_HIP_ERR_ARG, "bad dense operand or operator passed to comet_hip_eltwise_csr_dense_dense");
    if (a->nnz == 0)
        return COMET_HIP_OK;
    KernelTimer t("eltwise_mult_dense");
    eltwise_mult_dense_kernel<true><<<dim3((unsigned)ceil_div(a->nrows * 16, 256)), dim3(256), 0, stream()>>>(
        a->nrows, a->pos, a->crd, a->val, (const double *)d_dptr, ldd, (double *)c_dptr, ldc, op);
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}

// Dense (op) Dense over n elements (test/integration/semiring/eltwise_monoid*_DensexDense_oDense.ta).
__global__ void eltwise_dense_kernel(int64_t n, const double *__restrict__ a, const double *__restrict__ b,
                                     double *__restrict__ c, int op)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += step)
        c[i] = semiring_mult(op, a[i], b[i]);
}

extern "C" int comet_hip_eltwise_dense_f64(int64_t n, int64_t a_dptr, int64_t b_dptr, int64_t c_dptr, int op)
{
    COMET_CHK(ensure_init());
    if (n < 0 || (n > 0 && (!a_dptr || !b_dptr || !c_dptr)) || op < 0 || op > COMET_OP_DIV)
        return set_error(COMET_HIP_ERR_ARG, "bad arguments to comet_hip_eltwise_dense_f64");
    if (n == 0)
        return COMET_HIP_OK;
    KernelTimer t("eltwise_dense");
    const unsigned blocks = (unsigned)std::min<int64_t>(ceil_div(n, 256), (int64_t)num_cus() * 32);
    eltwise_dense_kernel<<<dim3(blocks), dim3(256), 0, stream()>>>(n, (const double *)a_dptr, (const double *)b_dptr,
                                                                  (double *)c_dptr, op);
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}

// Diagnostic: the vector registers per lane of the two kernels of the pattern-matrix masked sum, as the loaded code
// object has them.  The workgroup kernel (16 wavefronts, four to a SIMD) and one wavefront of the other kernel
// share a SIMD's 512 registers, allotted in eights: what a test holds them to.
extern "C" int comet_hip_debug_masked_sum_registers(int *workgroup_kernel, int *wavefront_kernel)
{
    COMET_CHK(ensure_init());
    if (!workgroup_kernel || !wavefront_kernel)
        return set_error(COMET_HIP_ERR_ARG, "null result pointer");
    hipFuncAttributes at;
    COMET_HIPCHK(hipFuncGetAttributes(&at, reinterpret_cast<const void *>(spgemm_masked_sum_iso_kernel)));
    *workgroup_kernel = at.numRegs;
    COMET_HIPCHK(hipFuncGetAttributes(&at, reinterpret_cast<const void *>(spgemm_masked_sum_small_iso_kernel)));
    *wavefront_kernel = at.numRegs;
    return COMET_HIP_OK;
}

// Diagnostic: where the fp64 sums of the dot-product kernel begin in its LDS, in 32-bit words, for a bitmap of
// `words` words (rounded up to what the host would ask for); lets a CPU-side test sweep the invariant "even".
extern "C" int comet_hip_debug_dot_table_words(int words)
{
    if (words < 1)
        words = 1;
    words = (int)ceil_div((int64_t)words, (int64_t)DT_WPT) * DT_WPT;
    return dot_table_words(words);
}
