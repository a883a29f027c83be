// LU factorisation with partial pivoting for MI355X (gfx950), the operation
// behind ulmBLAS's ulmblas_dgetrf / ulmblas_dlaswp (interfaces/lapack/C/
// getrf.cc:7-19, laswp.cc:7-18 -> ulmBLAS::getrf, ulmblas/lapack/getrf.tcc:
// 14-75, getf2.tcc:15-62, laswp.tcc:13-55).
//
// The reference factors column blocks of 64 left to right: unblocked panel
// (getf2: pivot search, row exchange, scaling, rank-1 update per column),
// row exchanges left and right of the panel (laswp), a unit lower solve for
// the block row of U (trlsm) and a rank-64 update of the trailing matrix
// (gemm).  Here the matrix stays in HBM for the whole factorisation and the
// same four ingredients are arranged for the GPU:
//   * the column range is split recursively, so that the trailing updates are
//     GEMMs with k = n/2, n/4, ... (matrix cores at full tile efficiency)
//     instead of 128 rank-64 updates that would each stream the whole
//     trailing matrix through HBM;
//   * the leaves are panels of up to 64 columns, factored by ONE launch of a
//     cooperative kernel: every workgroup keeps 256 rows of the panel in LDS,
//     and the workgroups agree on each column's pivot through a small
//     exchange area in HBM whose words say themselves which column they
//     belong to (one publication and one collection per column, no barrier);
//   * pivots, the info value and all control data stay on the device: the
//     whole factorisation is enqueued without a single host synchronisation.
// Pivoting is the reference's: first element of largest magnitude in the
// column, rows exchanged across the whole matrix, division through the
// reciprocal unless the pivot is below safe-min.
#include "internal.h"

#include <algorithm>
#include <cfloat>
#include <cmath>
#include <atomic>
#include <cstdio>
#include <mutex>
#include <string>

using namespace ulmgpu;

namespace ulmgpu {

constexpr int kPanelCols = 64;        // widest panel one launch factors
constexpr int kPanelRows = 256;       // rows per workgroup, one per thread of the first four wavefronts
constexpr int kPanelThreads = kPanelRows + 64;   // a fifth wavefront talks to the other workgroups
constexpr int kPanelPitch = kPanelCols + 1;   // LDS row pitch in doubles
constexpr int kMaxGroups = 256;       // workgroups of one panel launch (rows up to 65536)
constexpr long kSpinLimit = 1L << 24; // polls of one wait for the other workgroups before giving up (default)

// Exchange area of the panel kernel (device memory, part of the workspace).
struct PanelSlot {
    // Bits 0..62 the candidate's key (0 if the group has none), bit 63 the turn
    // of the slot -- bit 1 of the global column index, which flips every time
    // the slot is written again -- so that a reader sees from this one word
    // both that the slot is filled and with what.
    unsigned long long hdr;
    // Everything else carries the tag of its column (global column index + 1)
    // in the upper half of every 8-byte word, so that a reader can tell on its
    // own whether the word it got belongs to this column: no store here waits
    // for another one, and no reader needs a fence.
    unsigned long long rowtag;                  // lower half: panel-relative row of the candidate
    unsigned long long w[2 * kPanelCols];       // value i across the panel: lower half of its bits in w[2i], upper in w[2i+1]
};
// What the row exchanges of one panel do to every other column, worked out
// once by the panel kernel: lane l of a wave moving a column reads block row
// r0 + l and outside row ext_row[l] and stores into them what lane idx_b[l] /
// idx_e[l] read (flags say from which of the two reads, and whether to move at all).
struct SwapPlan {
    int idx_b[64], idx_e[64], ext_row[64], flags[64];
};
constexpr int kMoveB = 1, kMoveE = 2, kExtB = 4, kExtE = 8, kReadB = 16, kReadE = 32;

struct PanelWork {
    unsigned int failed;        // set when a wait gave up; every later wait falls through
    unsigned int pad[15];
    PanelSlot top[2];           // row c of the panel (the row the pivot row is exchanged with), by parity of c
    PanelSlot cand[2][kMaxGroups];
    SwapPlan plan;              // the finished panel's exchanges, for the kernel that applies them elsewhere
};

struct PanelArgs {
    double *A;          // element (j0, j0) of the matrix: top-left of the panel
    int64_t ldA;
    int rows, cols;     // panel extent: rows = m - j0, cols <= kPanelCols
    int j0;             // global index of the panel's first row/column (added to the pivots)
    int groups;         // workgroups of this launch
    int *piv;           // global pivot array (element j0 + c is written)
    int *info;          // 0, or 1 + index of the first zero pivot (global), kept if already set
    PanelWork *work;
    long spin_limit;    // polls of one wait before the workgroup gives up
};

// The limit handed to every launch; tests lower it to walk the give-up path.
std::atomic<long> g_spin_limit{kSpinLimit};
std::atomic<bool> g_simple_panels{false};   // testing: every panel takes the launches that wait for nobody
void lu_set_simple_panels(bool on) { g_simple_panels.store(on); }
thread_local bool g_simple_this_call = false;   // the host entry point's second attempt (getrf_host)
void lu_set_spin_limit(long polls) { g_spin_limit.store(polls >= 0 ? polls : kSpinLimit); }

__device__ __forceinline__ unsigned long long ld_agent(const unsigned long long *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ int ld_agent(const int *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent(unsigned long long *p, unsigned long long v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// A double as two tagged words (the reader puts the halves together again once both carry its tag).
__device__ __forceinline__ void put_tagged(unsigned long long *w, double v, unsigned tag)
{
    const unsigned long long b = (unsigned long long)__double_as_longlong(v), t = (unsigned long long)tag << 32;
    st_agent(w, (b & 0xffffffffull) | t);
    st_agent(w + 1, (b >> 32) | t);
}

// Order-preserving 63-bit key of a pivot candidate: 0 = not in play, 1 = a NaN
// below row c (never chosen over anything, ulmblas/level1/iamax.tcc:22-27 only
// replaces on a strict >), 2 + the bit pattern of |v| otherwise, and the key
// of +infinity for a NaN in row c itself (nothing compares greater than the
// starting value then).
__device__ __forceinline__ unsigned long long key_bits(double v, bool first)
{
    const double m = fabs(v);
    if (m != m) return first ? (unsigned long long)__double_as_longlong(HUGE_VAL) + 2ull : 1ull;
    return (unsigned long long)__double_as_longlong(m) + 2ull;
}
constexpr unsigned long long kTurnBit = 1ull << 63;

// One step of a wavefront scan through the data-parallel-primitive path of
// the vector ALU: lanes that have no source keep the identity `idle`.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ unsigned long long dpp_u64(unsigned long long v)
{
    int lo = (int)(unsigned)v, hi = (int)(unsigned)(v >> 32);
    lo = __builtin_amdgcn_update_dpp(0, lo, CTRL, ROW_MASK, 0xf, false);
    hi = __builtin_amdgcn_update_dpp(0, hi, CTRL, ROW_MASK, 0xf, false);
    return ((unsigned long long)(unsigned)hi << 32) | (unsigned)lo;
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_min_i32(int v)
{
    const int o = __builtin_amdgcn_update_dpp(0x7fffffff, v, CTRL, ROW_MASK, 0xf, false);
    return o < v ? o : v;
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ unsigned long long dpp_max_u64(unsigned long long v)
{
    const unsigned long long o = dpp_u64<CTRL, ROW_MASK>(v);
    return o > v ? o : v;
}

// Best pivot candidate of a wavefront: the largest key and, among the lanes
// that hold it, the smallest row (ulmblas/level1/iamax.tcc:22-27 keeps the
// first maximum).  Two inclusive scans (shift by 1, 2, 4, 8 within rows of 16
// lanes, then the row broadcasts) whose last lane holds the result; every
// lane returns it.  Cross-lane shuffles through the LDS crossbar would take
// eighteen dependent round trips here.
__device__ __forceinline__ void wave_best(unsigned long long &kb, int &row)
{
    unsigned long long m = kb;
    m = dpp_max_u64<0x111, 0xf>(m);      // row_shr:1
    m = dpp_max_u64<0x112, 0xf>(m);      // row_shr:2
    m = dpp_max_u64<0x114, 0xf>(m);      // row_shr:4
    m = dpp_max_u64<0x118, 0xf>(m);      // row_shr:8
    m = dpp_max_u64<0x142, 0xa>(m);      // row_bcast:15 into rows 1 and 3
    m = dpp_max_u64<0x143, 0xc>(m);      // row_bcast:31 into rows 2 and 3
    const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)m, 63);
    const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(m >> 32), 63);
    const unsigned long long best = ((unsigned long long)hi << 32) | lo;
    int r = (kb == best) ? row : 0x7fffffff;
    r = dpp_min_i32<0x111, 0xf>(r);
    r = dpp_min_i32<0x112, 0xf>(r);
    r = dpp_min_i32<0x114, 0xf>(r);
    r = dpp_min_i32<0x118, 0xf>(r);
    r = dpp_min_i32<0x142, 0xa>(r);
    r = dpp_min_i32<0x143, 0xc>(r);
    kb = best;
    row = __builtin_amdgcn_readlane(r, 63);
}

__device__ __forceinline__ void better(unsigned long long &kb, int &row, unsigned long long okb, int orow)
{
    if (okb > kb || (okb == kb && orow < row)) {
        kb = okb;
        row = orow;
    }
}

// The exchanges of rows r0 .. r0+cnt-1 with rows pv (lane i holds the pivot of
// step i, cnt <= 64) played on row numbers only, by one wavefront: on return
// lane l knows which block row / outside row it reads (r0 + l, ext_row) and
// which lane's reads end up there.
// The value lane `src` holds, for a lane number that is the same across the
// wavefront: a scalar read, not a trip through the LDS crossbar.
__device__ __forceinline__ int lane_value(int v, int src)
{
    return __builtin_amdgcn_readlane(v, __builtin_amdgcn_readfirstlane(src));
}

// The exchanges of rows r0 .. r0+cnt-1 with their pivot rows (cnt <= 64) played
// on row numbers only, by one wavefront.  State per lane l: cur_b, the row
// whose old content ends up in block row r0 + l; ext_row, an outside row that
// is touched (lane i takes the one first met in step i), and cur_e, the row
// whose old content ends up there.
struct SwapState {
    int cur_b, ext_row, cur_e;
};
__device__ __forceinline__ SwapState swap_start(int lane, int r0)
{
    return SwapState{r0 + lane, -1, -1};
}
// step i: block row r0 + i changes places with row p
__device__ __forceinline__ void swap_step(SwapState &s, int lane, int r0, int cnt, int i, int p)
{
    if (p == r0 + i) return;
    if (p >= r0 && p < r0 + cnt) {
        const int b = p - r0;
        const int va = lane_value(s.cur_b, i), vb = lane_value(s.cur_b, b);
        if (lane == i) s.cur_b = vb;
        if (lane == b) s.cur_b = va;
    } else {
        const unsigned long long hit = __ballot(s.ext_row == p);
        int slot = i;                       // a new outside row takes the slot of its step
        if (hit != 0) {
            slot = __ffsll((long long)hit) - 1;
        } else if (lane == i) {
            s.ext_row = p;
            s.cur_e = p;
        }
        const int va = lane_value(s.cur_b, i), ve = lane_value(s.cur_e, slot);
        if (lane == i) s.cur_b = ve;
        if (lane == slot) s.cur_e = va;
    }
}
// On return lane l knows which block row / outside row it reads (r0 + l,
// ext_row) and which lane's reads end up there.
__device__ __forceinline__ void swap_finish(const SwapState &s, int lane, int r0, int cnt, int &idx_b, int &idx_e,
                                            int &ext_row, int &flags)
{
    const int curB = s.cur_b, curE = s.cur_e, extRow = s.ext_row;
    // where each lane's new values come from: a block row (lane index) or an outside slot
    int idxB = curB - r0, idxE = curE - r0;
    bool extB = false, extE = false;
    if (curB < r0 || curB >= r0 + cnt) extB = true;
    if (curE < r0 || curE >= r0 + cnt) extE = true;
    for (int sidx = 0; sidx < 64; ++sidx) {
        const int er = lane_value(extRow, sidx);
        if (er < 0) continue;
        if (extB && er == curB) idxB = sidx;
        if (extE && er == curE) idxE = sidx;
    }
    const bool moveB = lane < cnt && curB != r0 + lane;
    const bool moveE = extRow >= 0 && curE != extRow;
    const bool readB = lane < cnt, readE = extRow >= 0;
    idx_b = idxB & 63;
    idx_e = idxE & 63;
    ext_row = extRow;
    flags = (moveB ? kMoveB : 0) | (moveE ? kMoveE : 0) | (extB ? kExtB : 0) | (extE ? kExtE : 0) |
            (readB ? kReadB : 0) | (readE ? kReadE : 0);
}
__device__ __forceinline__ void swap_plan(int lane, int r0, int cnt, int pv, int &idx_b, int &idx_e, int &ext_row,
                                          int &flags)
{
    SwapState s = swap_start(lane, r0);
    for (int i = 0; i < cnt; ++i) swap_step(s, lane, r0, cnt, i, lane_value(pv, i));
    swap_finish(s, lane, r0, cnt, idx_b, idx_e, ext_row, flags);
}

// ulmblas/lapack/getf2.tcc:15-62 on an (rows x cols) panel, cols <= 64.
// Workgroup g holds rows g*256 .. g*256+255 in LDS, thread t row g*256+t.
__global__ __launch_bounds__(kPanelThreads) void getf2_panel_kernel(PanelArgs a)
{
    extern __shared__ double lds[];
    double *xs = lds;                                   // [kPanelRows][kPanelPitch]
    double *us = xs + kPanelRows * kPanelPitch;         // pivot rows, two in turn
    double *ts = us + 2 * kPanelCols;                   // row c before the exchange
    __shared__ unsigned long long red_key[kPanelRows / 64];
    __shared__ int red_row[kPanelRows / 64];
    __shared__ int win_row;
    __shared__ int gave_up;          // a bounded wait ran out (here or in another group)

    const int t = threadIdx.x, g = blockIdx.x, G = a.groups;
    const int cols = a.cols;
    const int gr = g * kPanelRows + t;                  // my row, relative to the panel
    const bool worker = t < kPanelRows;                 // holds a row
    const int lane = t - kPanelRows;                    // >= 0: lane of the wavefront that communicates
    const bool have = worker && gr < a.rows;
    double *mine = xs + t * kPanelPitch;
    const double smin = DBL_MIN;                        // ulmblas/lapack/safemin.tcc:11-26 for double

    if (worker) {
        for (int c = 0; c < cols; ++c) mine[c] = have ? a.A[gr + c * a.ldA] : 0.0;
    }
    __syncthreads();

    if (t == 0) gave_up = 0;
    int first_zero = 0;
    // The elimination with pivot c is split: column c+1 is updated at once (the
    // next pivot search needs it), columns c+2.. are updated one step later,
    // while the fifth wavefront waits for the other groups' candidates.  `pend` says
    // such an update is outstanding, l_prev is this row's multiplier for it.
    bool pend = false;
    double l_prev = 0.0;
    SwapState plan = swap_start(lane, a.j0);
    for (int c = 0; c < cols; ++c) {
        double *usc = us + (c & 1) * kPanelCols;              // pivot row c
        const double *usp = us + ((c + 1) & 1) * kPanelCols;  // pivot row c-1, read by the outstanding update
        // 1. this group's candidate.  Rows above c are finished rows of U.
        //    A NaN never wins the reference's comparison unless it sits in
        //    row c itself, which is the starting value there.
        unsigned long long key = 0;         // 0: not in play
        int row = 0x7fffffff;
        if (have && gr >= c) {
            key = key_bits(mine[c], gr == c);
            row = gr;
        }
        wave_best(key, row);
        if ((t & 63) == 0 && worker) {
            red_key[t >> 6] = key;
            red_row[t >> 6] = row;
        }
        __syncthreads();
        // every thread folds the four wavefront results itself
        key = red_key[0];
        row = red_row[0];
        for (int w = 1; w < kPanelRows / 64; ++w) better(key, row, red_key[w], red_row[w]);

        // 2a. the fifth wavefront copies the candidate row and row c, lane i column i, and applies the
        //     outstanding update to these two rows itself, in place (their owners skip them below, so
        //     nobody has to wait for anybody here)
        double cand_v = 0.0, top_v = 0.0;
        if (lane >= 0 && lane < cols) {
            const bool upd = pend && lane > c;
            if (key != 0) {
                double *r = xs + (row - g * kPanelRows) * kPanelPitch;
                cand_v = r[lane];
                if (upd) {
                    cand_v = fma(-r[c - 1], usp[lane], cand_v);
                    r[lane] = cand_v;
                }
            }
            if (g == 0) {
                if (key != 0 && row == c) {
                    top_v = cand_v;
                } else {
                    double *r = xs + c * kPanelPitch;
                    top_v = r[lane];
                    if (upd) {
                        top_v = fma(-r[c - 1], usp[lane], top_v);
                        r[lane] = top_v;
                    }
                }
            }
        }

        // 2b. the pivot row (usc) and row c (ts) of the whole panel: the fifth wavefront publishes
        //     this group's candidate and collects everybody's; meanwhile the others apply the
        //     outstanding update to their rows.
        const int J = a.j0 + c;                       // global column: slots and turns carry over launches
        const int par = J & 1;
        const unsigned long long turn = ((unsigned long long)(J >> 1) & 1ull) << 63;
        const unsigned tag = (unsigned)J + 1u;
        if (lane >= 0 && G > 1) {
            // Header (key and the slot's turn) and tagged data go out together, as stores that
            // go straight through to memory; nothing waits for anything.
            PanelSlot *slot = &a.work->cand[par][g];
            if (lane == 0) st_agent(&slot->hdr, key | turn);
            if (key != 0 && lane < cols) put_tagged(&slot->w[2 * lane], cand_v, tag);
            if (lane == 0) st_agent(&slot->rowtag, (unsigned long long)(unsigned)row | ((unsigned long long)tag << 32));
            if (g == 0 && lane < cols) put_tagged(&a.work->top[par].w[2 * lane], top_v, tag);
        }
        if (pend && have && gr > c - 1 && gr != row && !(g == 0 && gr == c)) {
            // eight columns at a time, loads first: the LDS round trips overlap
            int q = c + 1;
            for (; q + 8 <= cols; q += 8) {
                double xv[8], uv[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    xv[e] = mine[q + e];
                    uv[e] = usp[q + e];
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) mine[q + e] = fma(-l_prev, uv[e], xv[e]);
            }
            for (; q < cols; ++q) mine[q] = fma(-l_prev, usp[q], mine[q]);
        }
        if (lane >= 0) {
            int prow = row;
            if (G > 1) {
                // Poll the headers of all groups, which is both the meeting point of the groups
                // and the delivery of their keys.  Every wait is bounded: a group that polls
                // spin_limit times without seeing the others marks the launch as failed and
                // every later wait falls through, so the grid always drains.  Lane i watches
                // groups i, i + 64, ...
                unsigned long long best = 0;
                int best_group = 0x7fffffff;
                const bool dead = *(volatile int *)&gave_up != 0;
                for (int base = 0; base < G; base += 64) {
                    const int og = base + lane;
                    bool ok = og >= G || dead;
                    unsigned long long h = 0;
                    long spins = 0;
                    for (;;) {
                        if (!ok) {
                            h = ld_agent(&a.work->cand[par][og].hdr);
                            ok = (h & kTurnBit) == turn;
                        }
                        if (__builtin_amdgcn_ballot_w64(!ok) == 0) break;
                        ++spins;
                        if (spins > a.spin_limit ||
                            ((spins & 63) == 0 &&
                             __hip_atomic_load(&a.work->failed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)) {
                            __hip_atomic_store(&a.work->failed, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            *(volatile int *)&gave_up = 1;
                            break;
                        }
                        __builtin_amdgcn_s_sleep(1);
                    }
                    if (og < G) better(best, best_group, h & ~kTurnBit, og);   // ties: the lowest group, i.e. row
                }
                wave_best(best, best_group);
                const int wg = (best_group >= 0 && best_group < G) ? best_group : 0;
                // the winner's row and row c, each word checked against this column's tag
                const PanelSlot *win = &a.work->cand[par][wg], *top = &a.work->top[par];
                double pv = 0.0, tv = 0.0;
                int r = c;
                bool okv = lane >= cols, okt = lane >= cols, okr = false;
                bool stop = *(volatile int *)&gave_up != 0;
                long spins = 0;
                while (!stop) {
                    // all five loads in flight together (lanes past the panel's width read along and ignore it)
                    const unsigned long long v0 = ld_agent(&win->w[2 * lane]), v1 = ld_agent(&win->w[2 * lane + 1]);
                    // row c is wanted only where the winning row lives (it takes that row's place there)
                    unsigned long long t0 = 0, t1 = 0;
                    if (wg == g) {
                        t0 = ld_agent(&top->w[2 * lane]);
                        t1 = ld_agent(&top->w[2 * lane + 1]);
                    }
                    const unsigned long long rt = ld_agent(&win->rowtag);
                    okv = lane >= cols || ((unsigned)(v0 >> 32) == tag && (unsigned)(v1 >> 32) == tag);
                    okt = lane >= cols || wg != g || ((unsigned)(t0 >> 32) == tag && (unsigned)(t1 >> 32) == tag);
                    okr = (unsigned)(rt >> 32) == tag;
                    pv = __longlong_as_double((long long)((v1 << 32) | (v0 & 0xffffffffull)));
                    tv = __longlong_as_double((long long)((t1 << 32) | (t0 & 0xffffffffull)));
                    r = (int)(unsigned)rt;
                    if (__builtin_amdgcn_ballot_w64(!(okv && okt && okr)) == 0) break;
                    ++spins;
                    if (spins > a.spin_limit ||
                        ((spins & 63) == 0 &&
                         __hip_atomic_load(&a.work->failed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)) {
                        __hip_atomic_store(&a.work->failed, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        *(volatile int *)&gave_up = 1;
                        stop = true;
                    }
                }
                if (lane < cols) {
                    usc[lane] = pv;
                    ts[lane] = tv;
                }
                prow = (okr && r >= c && r < a.rows) ? r : c;    // in range whatever a failed wait left behind
            } else if (lane < cols) {
                usc[lane] = cand_v;
                ts[lane] = top_v;
            }
            if (lane == 0) win_row = prow;
        }
        __syncthreads();

        // 3. exchange rows c and win_row across the panel (getf2.tcc:39-41); both copies carry
        //    every update up to pivot c-1, as the rows in LDS do by now
        const int prow = win_row;
        // group 0's fifth wavefront, idle until the next column's candidates are known, keeps the plan of
        // the panel's row exchanges up to date
        if (g == 0 && lane >= 0) swap_step(plan, lane, a.j0, cols, c, a.j0 + prow);
        if (prow != c && t < cols) {
            if (g == 0) xs[c * kPanelPitch + t] = usc[t];
            if (prow / kPanelRows == g) xs[(prow - g * kPanelRows) * kPanelPitch + t] = ts[t];
        }
        if (g == 0 && t == 0) a.piv[a.j0 + c] = a.j0 + prow;
        __syncthreads();

        // 4. scale the column below the diagonal (getf2.tcc:38-57) and eliminate in column c+1;
        //    the other columns follow in step 2b of the next round
        const double p = usc[c];
        pend = p != 0.0;
        if (pend) {
            if (have && gr > c) {
                double l = mine[c];
                if (fabs(p) >= smin) {
                    l *= 1.0 / p;
                } else {
                    l /= p;
                }
                mine[c] = l;
                l_prev = l;
                if (c + 1 < cols) mine[c + 1] = fma(-l, usc[c + 1], mine[c + 1]);
            }
        } else if (first_zero == 0) {
            first_zero = a.j0 + c + 1;
        }
    }
    __syncthreads();

    for (int c = 0; c < cols; ++c) {
        if (have) a.A[gr + c * a.ldA] = mine[c];
    }
    if (g == 0 && lane >= 0) {
        // what these exchanges do to the other columns of the matrix, for the kernel that follows
        int idx_b, idx_e, ext_row, flags;
        swap_finish(plan, lane, a.j0, cols, idx_b, idx_e, ext_row, flags);
        a.work->plan.idx_b[lane] = idx_b;
        a.work->plan.idx_e[lane] = idx_e;
        a.work->plan.ext_row[lane] = ext_row;
        a.work->plan.flags[lane] = flags;
    }
    if (g == 0 && t == 0) {
        if (first_zero != 0 && *a.info == 0) *a.info = first_zero;
        if (G > 1 && ld_agent(reinterpret_cast<const int *>(&a.work->failed)) != 0) *a.info = -1;
    }
}

// ---------------------------------------------------------------------------
// The same panel factorisation without any waiting between workgroups: three
// small launches per column (candidates per block of rows; choice, exchange of
// the two rows across the panel, pivot and info; scaling and elimination).
// For panels the cooperative kernel cannot take -- more rows than its
// workgroups can hold at the same time on this GPU -- at several microseconds
// per launch instead of one synchronisation per column.  The arithmetic is
// that of the cooperative kernel operation for operation (reciprocal of the
// pivot unless it is below safe-min, fused multiply-add in the elimination),
// so both give the same bits.
// ---------------------------------------------------------------------------
struct SimpleCand {
    unsigned long long key;
    int row, pad;
};
constexpr int kSimpleBlocks = 256;        // candidates per column (they live in the exchange area)
constexpr int kSimpleThreads = 256;

// best candidate of column c among the rows of this block (grid-stride over the rows c .. rows-1)
__global__ __launch_bounds__(kSimpleThreads) void simple_search_kernel(const double *A, int64_t ldA, int rows, int c,
                                                                        SimpleCand *cand)
{
    __shared__ unsigned long long red_key[kSimpleThreads / 64];
    __shared__ int red_row[kSimpleThreads / 64];
    unsigned long long key = 0;
    int row = 0x7fffffff;
    const double *x = A + (int64_t)c * ldA;
    for (int64_t r = (int64_t)c + blockIdx.x * blockDim.x + threadIdx.x; r < rows; r += (int64_t)gridDim.x * blockDim.x) {
        unsigned long long k2 = key_bits(x[r], r == c);
        better(key, row, k2, (int)r);
    }
    wave_best(key, row);
    if ((threadIdx.x & 63) == 0) {
        red_key[threadIdx.x >> 6] = key;
        red_row[threadIdx.x >> 6] = row;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kSimpleThreads / 64; ++w) better(key, row, red_key[w], red_row[w]);
        cand[blockIdx.x].key = key;
        cand[blockIdx.x].row = row;
    }
}

// one workgroup: the pivot of column c from the blocks' candidates, the exchange of rows c and
// pivot across the panel (getf2.tcc:39-41), the pivot entry and info (getf2.tcc:51-53)
__global__ __launch_bounds__(64) void simple_pivot_kernel(double *A, int64_t ldA, int rows, int cols, int c, int j0,
                                                          const SimpleCand *cand, int ncand, int *piv, int *info,
                                                          double *pivot_value)
{
    const int lane = threadIdx.x;
    unsigned long long key = 0;
    int row = 0x7fffffff;
    for (int i = lane; i < ncand; i += 64) better(key, row, cand[i].key, cand[i].row);
    wave_best(key, row);
    const int p = (key != 0 && row >= c && row < rows) ? row : c;
    if (p != c) {
        for (int q = lane; q < cols; q += 64) {
            double *col = A + (int64_t)q * ldA;
            const double v = col[c];
            col[c] = col[p];
            col[p] = v;
        }
    }
    __syncthreads();
    if (lane == 0) {
        piv[j0 + c] = j0 + p;
        const double pv = A[(int64_t)c * ldA + c];
        *pivot_value = pv;
        if (pv == 0.0 && *info == 0) *info = j0 + c + 1;
    }
}

// rows below c: multiplier, then elimination in the columns to the right (getf2.tcc:38-57)
__global__ __launch_bounds__(kSimpleThreads) void simple_update_kernel(double *A, int64_t ldA, int rows, int cols, int c,
                                                                        const double *pivot_value)
{
    const double p = *pivot_value;
    if (p == 0.0) return;
    const int64_t r = (int64_t)c + 1 + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= rows) return;
    double l = A[(int64_t)c * ldA + r];
    if (fabs(p) >= DBL_MIN) {
        l *= 1.0 / p;
    } else {
        l /= p;
    }
    A[(int64_t)c * ldA + r] = l;
    for (int q = c + 1; q < cols; ++q) {
        double *col = A + (int64_t)q * ldA;
        col[r] = fma(-l, col[c], col[r]);
    }
}

// ulmblas/lapack/laswp.tcc:13-55 on column-major data: rows i = k1 .. k2-1 in
// turn (backwards when inc_piv < 0) are exchanged with rows piv[i*inc_piv],
// over n columns; one thread walks one column.
__global__ void laswp_kernel(int n, double *A, int64_t ldA, int k1, int k2, const int *piv, int inc_piv)
{
    const int64_t col = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (col >= n) return;
    double *x = A + col * ldA;
    if (inc_piv > 0) {
        for (int i = k1; i < k2; ++i) {
            const int ip = piv[(int64_t)i * inc_piv];
            if (ip != i) {
                const double v = x[i];
                x[i] = x[ip];
                x[ip] = v;
            }
        }
    } else {
        for (int i = k2 - 1; i >= k1; --i) {
            const int ip = piv[(int64_t)i * inc_piv];
            if (ip != i) {
                const double v = x[i];
                x[i] = x[ip];
                x[ip] = v;
            }
        }
    }
}

// The same exchanges for up to 64 consecutive pivots with unit stride, as one
// gather/scatter pass: rows r0 .. r0+cnt-1 in turn are exchanged with rows
// piv[r0+i].  Walking the exchanges one after the other costs cnt dependent
// memory round trips per column; instead every wave first plays the sequence
// on row numbers only (in registers: lane l tracks block row r0+l and the
// l-th outside row that gets touched) and then moves each column's at most
// 2*cnt affected elements in one step, lanes along the rows.  Columns
// [hole_begin, hole_begin + hole_len) are skipped (the panel that produced
// the pivots has exchanged its own rows already).
__global__ __launch_bounds__(256) void laswp_block_kernel(int ncols, double *A, int64_t ldA, int r0, int cnt,
                                                          const int *piv, int hole_begin, int hole_len,
                                                          const SwapPlan *plan)
{
    const int lane = threadIdx.x & 63;
    int idxB, idxE, extRow, flags;
    if (plan) {                     // worked out by the kernel that chose the pivots
        idxB = plan->idx_b[lane];
        idxE = plan->idx_e[lane];
        extRow = plan->ext_row[lane];
        flags = plan->flags[lane];
    } else {
        const int pv = (lane < cnt) ? piv[r0 + lane] : 0;
        swap_plan(lane, r0, cnt, pv, idxB, idxE, extRow, flags);
    }
    const bool moveB = flags & kMoveB, moveE = flags & kMoveE, extB = flags & kExtB, extE = flags & kExtE;
    const bool readB = flags & kReadB, readE = flags & kReadE;

    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int waves = (gridDim.x * blockDim.x) >> 6;
    // four columns in flight per wave: their loads are issued before the first store
    constexpr int U = 4;
    for (int c0 = wave * U; c0 < ncols; c0 += waves * U) {
        double *x[U];
        double xB[U], xE[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int cc = c0 + u < ncols ? c0 + u : ncols - 1;     // a repeated last column is read, not written
            const int c = cc < hole_begin ? cc : cc + hole_len;
            x[u] = A + (int64_t)c * ldA;
            xB[u] = readB ? x[u][r0 + lane] : 0.0;
            xE[u] = readE ? x[u][extRow] : 0.0;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const double fromB_B = __shfl(xB[u], idxB & 63), fromE_B = __shfl(xE[u], idxB & 63);
            const double fromB_E = __shfl(xB[u], idxE & 63), fromE_E = __shfl(xE[u], idxE & 63);
            if (c0 + u < ncols) {
                if (moveB) x[u][r0 + lane] = extB ? fromE_B : fromB_B;
                if (moveE) x[u][extRow] = extE ? fromE_E : fromB_E;
            }
        }
    }
}

// dst (cols x rows, leading dimension ldd) <- transpose of src (rows x cols, lds)
__global__ void transpose_kernel(int rows, int cols, const double *src, int64_t lds_, double *dst, int64_t ldd)
{
    __shared__ double tile[32][33];
    const int bi = blockIdx.x * 32, bj = blockIdx.y * 32;
    for (int jj = threadIdx.y; jj < 32; jj += blockDim.y) {
        const int i = bi + threadIdx.x, j = bj + jj;
        if (i < rows && j < cols) tile[jj][threadIdx.x] = src[i + j * lds_];
    }
    __syncthreads();
    for (int ii = threadIdx.y; ii < 32; ii += blockDim.y) {
        const int j = bj + threadIdx.x, i = bi + ii;
        if (i < rows && j < cols) dst[j + i * ldd] = tile[threadIdx.x][ii];
    }
}

// Start of a factorisation: no failure, info = 0, every slot's header one turn
// behind what its first reader will wait for (columns 0 and 1 wait for turn
// 0), and no tagged word that a column of this factorisation could take for
// its own (tags start at 1).
constexpr int kResetBlocks = 32;
__global__ void lu_reset_kernel(PanelWork *w, int *info)
{
    const int t = blockIdx.x * blockDim.x + threadIdx.x, nt = gridDim.x * blockDim.x;
    if (t == 0) {
        w->failed = 0;
        if (info) *info = 0;
    }
    constexpr int kWords = (int)(sizeof(PanelSlot) / sizeof(unsigned long long));
    for (int i = t; i < (2 * kMaxGroups + 2) * kWords; i += nt) {
        const int s = i / kWords, e = i % kWords;
        PanelSlot *slot = s < 2 ? &w->top[s] : &w->cand[(s - 2) / kMaxGroups][(s - 2) % kMaxGroups];
        reinterpret_cast<unsigned long long *>(slot)[e] = (e == 0) ? kTurnBit : 0ull;
    }
}

// Exchanges of rows r0 .. r0+cnt-1 (cnt <= 64, pivots at unit stride) over
// `ncols` columns counted without the hole.
int launch_laswp_block(int ncols, double *dA, int64_t ldA, int r0, int cnt, const int *dPiv, int hole_begin,
                       int hole_len, hipStream_t stream, const SwapPlan *plan = nullptr)
{
    if (ncols <= 0 || cnt <= 0) return ULMBLAS_GPU_OK;
    const int waves = std::min((ncols + 3) / 4, 8192);
    hipLaunchKernelGGL(laswp_block_kernel, dim3((waves + 3) / 4), dim3(256), 0, stream, ncols, dA, ldA, r0, cnt, dPiv,
                       hole_begin, hole_len, plan);
    HIP_TRY(hipGetLastError());
    return ULMBLAS_GPU_OK;
}

int launch_laswp(int n, double *dA, int64_t ldA, int k1, int k2, const int *dPiv, int inc_piv, hipStream_t stream)
{
    if (n <= 0 || k2 <= k1 || inc_piv == 0) return ULMBLAS_GPU_OK;
    if (inc_piv == 1) {
        for (int r0 = k1; r0 < k2; r0 += 64) {
            const int rc = launch_laswp_block(n, dA, ldA, r0, std::min(64, k2 - r0), dPiv, n, 0, stream);
            if (rc) return rc;
        }
        return ULMBLAS_GPU_OK;
    }
    const int threads = 128;
    hipLaunchKernelGGL(laswp_kernel, dim3((n + threads - 1) / threads), dim3(threads), 0, stream, n, dA, ldA, k1, k2,
                       dPiv, inc_piv);
    HIP_TRY(hipGetLastError());
    return ULMBLAS_GPU_OK;
}

constexpr size_t kPanelLdsBytes = (size_t)(kPanelRows * kPanelPitch + 3 * kPanelCols) * sizeof(double);

// Workgroups of the panel kernel that the current device holds at the same time when nothing
// else runs on it (0 with g_last_error set if that cannot be found out).  Asked once per device.
int panel_capacity()
{
    static std::mutex mu;
    static int cached[64];
    int dev = -1;
    if (!hip_ok(hipGetDevice(&dev), "hipGetDevice") || dev < 0 || dev >= 64) return 0;
    std::lock_guard<std::mutex> lock(mu);
    if (cached[dev] == 0) {
        int per_cu = 0, cus = 0;
        if (!hip_ok(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, getf2_panel_kernel, kPanelThreads,
                                                                 kPanelLdsBytes),
                    "hipOccupancyMaxActiveBlocksPerMultiprocessor(getf2_panel_kernel)") ||
            !hip_ok(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev),
                    "hipDeviceGetAttribute(multiprocessor count)")) return 0;
        cached[dev] = per_cu * cus;
        if (cached[dev] <= 0) {
            g_last_error = "dgetrf: the panel kernel does not fit on this GPU";
            return 0;
        }
    }
    return cached[dev];
}

struct LuPlan {
    int m, n, mn;
    double *A;
    int ldA;
    int *piv, *info;
    PanelWork *work;
    hipStream_t stream;

    double *at(int i, int j) const { return A + i + (int64_t)j * ldA; }

    int panel(int j0, int cols)
    {
        static std::once_flag once;
        static hipError_t attr_status = hipSuccess;
        std::call_once(once, [&] {
            attr_status = hipFuncSetAttribute(reinterpret_cast<const void *>(getf2_panel_kernel),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)kPanelLdsBytes);
        });
        HIP_TRY(attr_status);
        PanelArgs a;
        a.A = at(j0, j0);
        a.ldA = ldA;
        a.rows = m - j0;
        a.cols = cols;
        a.j0 = j0;
        a.groups = (a.rows + kPanelRows - 1) / kPanelRows;
        a.piv = piv;
        a.info = info;
        a.work = work;
        a.spin_limit = g_spin_limit.load();
        // The workgroups of the panel kernel wait for one another, so all of them must be on the
        // GPU at the same time.  What can be known before the launch is whether the GPU could
        // hold them if it were otherwise idle (a GPU that other work keeps busy may still hold
        // fewer: then the bounded waits run out and the factorisation reports info = -1).  A
        // panel with more rows than that takes the launches that wait for nobody.
        const int capacity = panel_capacity();
        if (capacity <= 0) return ULMBLAS_GPU_HIP_ERROR;
        if (a.groups > std::min(capacity, kMaxGroups) || g_simple_panels.load() || g_simple_this_call)
            return simple_panel(j0, cols);
        hipLaunchKernelGGL(getf2_panel_kernel, dim3(a.groups), dim3(kPanelThreads), kPanelLdsBytes, stream, a);
        HIP_TRY(hipGetLastError());
        // the panel's row exchanges on every other column of the matrix, left and right (getrf.tcc:52-58)
        return launch_laswp_block(n - cols, A, ldA, j0, cols, piv, j0, cols, stream, &work->plan);
    }

    int simple_panel(int j0, int cols)
    {
        double *P = at(j0, j0);
        const int rows = m - j0;
        // the exchange area is free (no cooperative kernel runs in this factorisation's stream now):
        // candidates and the pivot's value live in its slots
        SimpleCand *cand = reinterpret_cast<SimpleCand *>(&work->cand[0][0]);
        double *pivot_value = reinterpret_cast<double *>(&work->top[0]);
        static_assert(sizeof(SimpleCand) * kSimpleBlocks <= sizeof(work->cand), "candidates fit the exchange area");
        for (int c = 0; c < cols; ++c) {
            const int left = rows - c;
            const int blocks = std::max(1, std::min(kSimpleBlocks, (left + kSimpleThreads - 1) / kSimpleThreads));
            hipLaunchKernelGGL(simple_search_kernel, dim3(blocks), dim3(kSimpleThreads), 0, stream, P, (int64_t)ldA, rows,
                               c, cand);
            hipLaunchKernelGGL(simple_pivot_kernel, dim3(1), dim3(64), 0, stream, P, (int64_t)ldA, rows, cols, c, j0,
                               cand, blocks, piv, info, pivot_value);
            if (left > 1) {
                hipLaunchKernelGGL(simple_update_kernel, dim3((left - 1 + kSimpleThreads - 1) / kSimpleThreads),
                                   dim3(kSimpleThreads), 0, stream, P, (int64_t)ldA, rows, cols, c, pivot_value);
            }
        }
        HIP_TRY(hipGetLastError());
        // the exchange area as a later cooperative panel expects it
        hipLaunchKernelGGL(lu_reset_kernel, dim3(kResetBlocks), dim3(256), 0, stream, work, static_cast<int *>(nullptr));
        HIP_TRY(hipGetLastError());
        return launch_laswp_block(n - cols, A, ldA, j0, cols, piv, j0, cols, stream, nullptr);
    }

    // Factor columns [j0, j0 + w) of the rows j0 .. m-1 (w <= mn - j0).
    int run(int j0, int w)
    {
        if (w <= kPanelCols) return panel(j0, w);
        const int w1 = ((w / 2 + kPanelCols - 1) / kPanelCols) * kPanelCols, w2 = w - w1;
        int rc;
        if ((rc = run(j0, w1))) return rc;
        // U12 = inv(L11) A12; A22 -= A21 U12 (every panel has applied its row exchanges to all columns already)
        if ((rc = trsm_device<double>(false, true, false, true, w1, w2, 1.0, at(j0, j0), ldA, at(j0, j0 + w1), ldA,
                                      stream))) return rc;
        if (m - j0 - w1 > 0) {
            if ((rc = gemm_device<double>(false, false, m - j0 - w1, w2, w1, -1.0, at(j0 + w1, j0), ldA,
                                          at(j0, j0 + w1), ldA, 1.0, at(j0 + w1, j0 + w1), ldA, stream))) return rc;
        }
        return run(j0 + w1, w2);
    }
};

}  // namespace ulmgpu

namespace ulmgpu {

// Column-major LU on device memory.  `work` holds at least
// ulmblas_gpu_dgetrf_worksize() bytes; dPiv min(m, n) ints; dInfo one int.
int getrf_device(int m, int n, double *dA, int ldA, int *dPiv, int *dInfo, void *work, hipStream_t stream)
{
    if (m < 0 || n < 0 || ldA < std::max(1, m)) {
        g_last_error = "invalid size or leading dimension";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    if (!dInfo || !work || ((m > 0 && n > 0) && (!dA || !dPiv))) {
        g_last_error = "null operand";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    if (reinterpret_cast<uintptr_t>(work) % 16 != 0) {
        g_last_error = "workspace must be 16-byte aligned";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    LuPlan p;
    p.m = m;
    p.n = n;
    p.mn = std::min(m, n);
    p.A = dA;
    p.ldA = ldA;
    p.piv = dPiv;
    p.info = dInfo;
    p.work = static_cast<PanelWork *>(work);
    p.stream = stream;
    hipLaunchKernelGGL(lu_reset_kernel, dim3(kResetBlocks), dim3(256), 0, stream, p.work, dInfo);
    HIP_TRY(hipGetLastError());
    if (m == 0 || n == 0) return ULMBLAS_GPU_OK;       // getrf.tcc:25-27
    int rc;
    if ((rc = p.run(0, p.mn))) return rc;
    if (n > p.mn) {
        // wide matrix: the columns right of the square part
        if ((rc = trsm_device<double>(false, true, false, true, p.mn, n - p.mn, 1.0, dA, ldA, p.at(0, p.mn), ldA,
                                      stream))) return rc;
    }
    return ULMBLAS_GPU_OK;
}

// ---------------------------------------------------------------------------
// The factorisation for callers that cannot allocate device memory (code under
// HIP graph capture, serving loops, harnesses that forbid hipMalloc): the
// exchange area of the panel kernel lives in a file-scope device array instead
// of a caller's workspace.  Every GPU holds its own copy of the array at its
// own address; the address is looked up once per device and handed to the
// kernels like any other workspace pointer.
// ---------------------------------------------------------------------------
constexpr size_t kStaticWorkBytes = (sizeof(PanelWork) + 255) / 256 * 256;
static __device__ __align__(256) unsigned char scratch[kStaticWorkBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void *g_scratch_ptr[kMaxDevices];       // per device: where `scratch` lives there (guarded by g_scratch_mu)

// Device address of `scratch` on the current device (null with g_last_error set on failure).
void *static_work_of_current_device()
{
    int dev = -1;
    if (!hip_ok(hipGetDevice(&dev), "hipGetDevice")) return nullptr;
    if (dev < 0 || dev >= kMaxDevices) {
        g_last_error = "device index out of range";
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        if (!hip_ok(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return nullptr;
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}

// pivots, exchange area + info word and the transposed copy of the row-major entry: per host context
int lu_host_reserve(HostContext &c, size_t npiv, size_t scratch_bytes)
{
    if (!c.lu_work) {
        HIP_TRY(HostContext::device_alloc(&c.lu_work, sizeof(PanelWork) + 64));
        c.lu_info = reinterpret_cast<int *>(static_cast<char *>(c.lu_work) + sizeof(PanelWork));
    }
    if (npiv > c.lu_piv_cap) {
        if (c.lu_piv) HIP_TRY(hipFree(c.lu_piv));
        c.lu_piv = nullptr;
        c.lu_piv_cap = 0;
        HIP_TRY(HostContext::device_alloc(reinterpret_cast<void **>(&c.lu_piv), (npiv + 1024) * sizeof(int)));
        c.lu_piv_cap = npiv + 1024;
    }
    if (scratch_bytes > c.lu_scratch_cap) {
        if (c.lu_scratch) HIP_TRY(hipFree(c.lu_scratch));
        c.lu_scratch = nullptr;
        c.lu_scratch_cap = 0;
        HIP_TRY(HostContext::device_alloc(&c.lu_scratch, scratch_bytes + scratch_bytes / 4));
        c.lu_scratch_cap = scratch_bytes + scratch_bytes / 4;
    }
    return ULMBLAS_GPU_OK;
}

// interfaces/lapack/C/getrf.cc:7-19 on host pointers.  `rows x cols` is the
// matrix the factorisation sees: (m, n) with strides (1, ldA) for
// column-major, (n, m) with strides (ldA, 1) for the row-major branch, which
// is served by factoring the transposed copy.
int getrf_host(bool row_major, int m, int n, double *A, int ldA, int *piv, int *info_out)
{
    *info_out = 0;
    if (m <= 0 || n <= 0) return ULMBLAS_GPU_OK;
    return with_context([&](HostContext &c) -> int {
    int rc = c.ensure_stream();
    if (rc) return rc;
    const int rows = row_major ? n : m, cols = row_major ? m : n;   // of the factored matrix
    const int mn = std::min(rows, cols);
    // what lies in memory, seen column-major: srows x scols with leading dimension ldA
    const int srows = row_major ? cols : rows, scols = row_major ? rows : cols;
    if ((rc = c.reserve(2, (size_t)srows * scols * sizeof(double)))) return rc;
    if ((rc = lu_host_reserve(c, (size_t)mn, row_major ? (size_t)rows * cols * sizeof(double) : 0))) return rc;
    double *dS = static_cast<double *>(c.buf[2]);
    // a large matrix travels through the pinned rings
    const bool streamed = streams_transfers(c, 2 * (size_t)srows * scols * sizeof(double), (size_t)srows * sizeof(double));
    if ((rc = host_upload<double>(c, streamed, A, ldA, dS, srows, srows, scols))) return rc;
    double *dF = dS;
    if (row_major) {
        dF = static_cast<double *>(c.lu_scratch);
        hipLaunchKernelGGL(transpose_kernel, dim3((srows + 31) / 32, (scols + 31) / 32), dim3(32, 8), 0, c.stream,
                           srows, scols, dS, (int64_t)srows, dF, (int64_t)rows);
        HIP_TRY(hipGetLastError());
    }
    // The status is read before anything travels back.  If the panel kernel's workgroups could not
    // meet (the GPU holds other work: every bounded wait ran out, info = -1) the matrix goes up
    // again and is factored by the launches that wait for nobody -- slower, the same arithmetic,
    // the same pivots.  Should that fail too the caller's matrix and pivots stay as they were.
    for (int attempt = 0; attempt < 2; ++attempt) {
        if (attempt == 1) {
            if ((rc = host_upload<double>(c, streamed, A, ldA, dS, srows, srows, scols))) return rc;
            if (row_major) {
                hipLaunchKernelGGL(transpose_kernel, dim3((srows + 31) / 32, (scols + 31) / 32), dim3(32, 8), 0, c.stream,
                                   srows, scols, dS, (int64_t)srows, dF, (int64_t)rows);
                HIP_TRY(hipGetLastError());
            }
        }
        g_simple_this_call = attempt == 1;
        rc = getrf_device(rows, cols, dF, rows, c.lu_piv, c.lu_info, c.lu_work, c.stream);
        g_simple_this_call = false;
        if (rc) return rc;
        HIP_TRY(hipMemcpyAsync(info_out, c.lu_info, sizeof(int), hipMemcpyDeviceToHost, c.stream));
        HIP_TRY(hipStreamSynchronize(c.stream));
        if (*info_out >= 0) break;
    }
    if (*info_out < 0) {
        g_last_error = "dgetrf: the factorisation could not be completed on the device; A and piv are unchanged";
        return ULMBLAS_GPU_HIP_ERROR;
    }
    if (row_major) {
        hipLaunchKernelGGL(transpose_kernel, dim3((rows + 31) / 32, (cols + 31) / 32), dim3(32, 8), 0, c.stream, rows,
                           cols, dF, (int64_t)rows, dS, (int64_t)srows);
        HIP_TRY(hipGetLastError());
    }
    HIP_TRY(hipMemcpyAsync(piv, c.lu_piv, (size_t)mn * sizeof(int), hipMemcpyDeviceToHost, c.stream));
    if ((rc = host_download<double>(c, streamed, dS, srows, A, ldA, srows, scols))) return rc;
    HIP_TRY(hipStreamSynchronize(c.stream));
    return ULMBLAS_GPU_OK;
    });
}

// interfaces/lapack/C/laswp.cc:7-18 on host pointers: only the rows the
// exchanges can touch travel to the device.
int laswp_host(int n, double *A, int ldA, int k1, int k2, const int *piv, int inc_piv)
{
    if (n <= 0 || inc_piv == 0 || k2 <= k1) return ULMBLAS_GPU_OK;
    // entries piv[i*inc_piv], i = k1 .. k2-1, whatever the sign of inc_piv
    const int64_t lo = std::min((int64_t)k1 * inc_piv, (int64_t)(k2 - 1) * inc_piv);
    const int64_t hi = std::max((int64_t)k1 * inc_piv, (int64_t)(k2 - 1) * inc_piv);
    int top = k2 - 1;
    for (int i = k1; i < k2; ++i) {
        const int ip = piv[(int64_t)i * inc_piv];
        if (ip < 0) {
            g_last_error = "dlaswp: negative row index";
            return ULMBLAS_GPU_BAD_ARGUMENT;
        }
        top = std::max(top, ip);
    }
    const int rows = top + 1;
    return with_context([&](HostContext &c) -> int {
    int rc = c.ensure_stream();
    if (rc) return rc;
    if ((rc = c.reserve(2, (size_t)rows * n * sizeof(double)))) return rc;
    if ((rc = lu_host_reserve(c, (size_t)(hi - lo + 1), 0))) return rc;
    double *dA = static_cast<double *>(c.buf[2]);
    if ((rc = copy_window<double>(dA, (size_t)rows * sizeof(double), A, (size_t)ldA * sizeof(double), rows, n,
                                  hipMemcpyHostToDevice, c.stream))) return rc;
    HIP_TRY(hipMemcpyAsync(c.lu_piv, piv + lo, (size_t)(hi - lo + 1) * sizeof(int), hipMemcpyHostToDevice, c.stream));
    if ((rc = launch_laswp(n, dA, rows, k1, k2, c.lu_piv - lo, inc_piv, c.stream))) return rc;
    if ((rc = copy_window<double>(A, (size_t)ldA * sizeof(double), dA, (size_t)rows * sizeof(double), rows, n,
                                  hipMemcpyDeviceToHost, c.stream))) return rc;
    HIP_TRY(hipStreamSynchronize(c.stream));
    return ULMBLAS_GPU_OK;
    });
}

}  // namespace ulmgpu

extern "C" {

int ulmblas_dgetrf(enum CBLAS_ORDER order, int m, int n, double *A, int ldA, int *piv)
{
    int info = 0;
    const int rc = getrf_host(order != CblasColMajor, m, n, A, ldA, piv, &info);
    report_host_status("ulmblas_dgetrf", rc, nullptr);
    if (rc != ULMBLAS_GPU_OK) return -1;
    return info;
}

void ulmblas_dlaswp(int n, double *A, int ldA, int k1, int k2, int *piv, int incPiv)
{
    const int rc = laswp_host(n, A, ldA, k1, k2, piv, incPiv);
    report_host_status("ulmblas_dlaswp", rc, nullptr);
}

int ATL_dgetrf(enum CBLAS_ORDER order, int m, int n, double *A, int ldA, int *piv)
{
    return ulmblas_dgetrf(order, m, n, A, ldA, piv);
}

void ATL_dlaswp(int n, double *A, int ldA, int k1, int k2, int *piv, int incPiv)
{
    ulmblas_dlaswp(n, A, ldA, k1, k2, piv, incPiv);
}

long ulmblas_gpu_dgetrf_worksize(void) { return (long)sizeof(PanelWork); }

int ulmblas_gpu_dgetrf(int m, int n, double *dA, int ldA, int *dPiv, int *dInfo, void *work, void *stream)
{
    return getrf_device(m, n, dA, ldA, dPiv, dInfo, work, static_cast<hipStream_t>(stream));
}

int ulmblas_gpu_dgetrf_static(int m, int n, double *dA, int ldA, int *dPiv, int *dInfo, void *stream)
{
    if (m > ULMBLAS_GPU_DGETRF_STATIC_MAX || n > ULMBLAS_GPU_DGETRF_STATIC_MAX) {
        g_last_error = "ulmblas_gpu_dgetrf_static: at most 65536 rows and 65536 columns";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    void *work = static_work_of_current_device();
    if (!work) return ULMBLAS_GPU_HIP_ERROR;
    InlineStrips no_side_streams;     // the updates' ragged strips go to the caller's stream: nothing is created
    return getrf_device(m, n, dA, ldA, dPiv, dInfo, work, static_cast<hipStream_t>(stream));
}

int ulmblas_gpu_dlaswp(int n, double *dA, int ldA, int k1, int k2, const int *dPiv, int incPiv, void *stream)
{
    if (n < 0 || ldA < 1) {
        g_last_error = "invalid size or leading dimension";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    return launch_laswp(n, dA, ldA, k1, k2, dPiv, incPiv, static_cast<hipStream_t>(stream));
}

}  // extern "C"
