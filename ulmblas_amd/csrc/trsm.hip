// Triangular solve with multiple right-hand sides for MI355X (gfx950):
// B <- alpha * inv(op(A)) * B  (left)  or  B <- alpha * B * inv(op(A))  (right),
// the operation behind ulmBLAS's dtrsm_ / strsm_ / cblas_?trsm
// (interfaces/blas/F77/trsm.cc, interfaces/blas/C/trsm.cc -> ulmBLAS::trlsm,
// ulmblas/level3/trlsm.tcc:16-91, and ulmBLAS::trusm, trusm.tcc:18-100).
//
// The reference walks MC-row blocks: solve the diagonal block against the
// packed B (mtrlsm / utrlsm), then update all rows still to be solved with one
// mgemm.  Here the same two ingredients are arranged for a GPU: the triangle
// is split recursively, the off-diagonal part of every split is one call of
// the matrix-core GEMM (large k near the root, so most flops run at GEMM
// speed), and what is left on the diagonal are blocks of up to 512 unknowns,
// each one launch: kLeaf x kLeaf triangles solved by substitution (several
// lanes per right-hand side, the triangle held in LDS) with matrix
// instructions between them, the right-hand sides resident in LDS, 256
// unknowns at a time.  Like the
// reference's trlspack the substitution multiplies by the reciprocal of the
// diagonal instead of dividing.
#include "internal.h"

#include <algorithm>
#include <atomic>
#include <cctype>
#include <cstdio>
#include <type_traits>

using namespace ulmgpu;

namespace ulmgpu {

constexpr int kLeaf = 64;          // order of the triangles solved by substitution
constexpr int kLeafVecs = 64;      // right-hand sides per workgroup, four lanes each
constexpr int kLoadThreads = 256;  // threads of a workgroup

// f(integral_constant<int, I>) for I = BEGIN .. END-1, expanded at compile time
template <int BEGIN, int END, class F>
__device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (BEGIN < END) {
        f(std::integral_constant<int, BEGIN>{});
        static_for<BEGIN + 1, END>(f);
    }
}

// Compiler fence on one register value: what produces v is scheduled before
// this point, what consumes it after.
template <typename T>
__device__ __forceinline__ void pin(T &v)
{
    asm volatile("" : "+v"(v));
}


template <typename T>
struct LeafArgs {
    const T *A;          // top-left element of the diagonal block
    int64_t a_si, a_sl;  // M[i][l] = A[i*a_si + l*a_sl] for the system matrix M (lower triangular after the
                         // optional reversal of both indices)
    T *B;                // first right-hand side
    int64_t b_si, b_sv;  // element i of vector v at B[i*b_si + v*b_sv]
    int nb;              // order of this block, <= kLeaf
    int nvec;            // number of right-hand sides
    int reversed;        // solve from the last unknown to the first (M upper triangular)
    int unit;            // unit diagonal: A's diagonal is not read
    T alpha;
};

// The value lane Q of every group of four lanes holds, handed to all four
// (a data-parallel-primitive move inside the vector ALU, no LDS round trip).
template <int Q>
__device__ __forceinline__ double quad_bcast(double v)
{
    constexpr int ctrl = Q | (Q << 2) | (Q << 4) | (Q << 6);      // quad_perm:[Q,Q,Q,Q]
    int lo = __double2loint(v), hi = __double2hiint(v);
    lo = __builtin_amdgcn_update_dpp(lo, lo, ctrl, 0xf, 0xf, true);
    hi = __builtin_amdgcn_update_dpp(hi, hi, ctrl, 0xf, 0xf, true);
    return __hiloint2double(hi, lo);
}
template <int Q>
__device__ __forceinline__ float quad_bcast(float v)
{
    constexpr int ctrl = Q | (Q << 2) | (Q << 4) | (Q << 6);
    const int b = __float_as_int(v);
    return __int_as_float(__builtin_amdgcn_update_dpp(b, b, ctrl, 0xf, 0xf, true));
}
// The same for groups of sixteen lanes (the rows of the data-parallel-primitive
// path): the value lane Q of every row holds, handed to the whole row.
template <int Q>
__device__ __forceinline__ double row_bcast(double v)
{
    constexpr int ctrl = 0x150 + Q;                               // row_newbcast:Q
    int lo = __double2loint(v), hi = __double2hiint(v);
    lo = __builtin_amdgcn_update_dpp(lo, lo, ctrl, 0xf, 0xf, true);
    hi = __builtin_amdgcn_update_dpp(hi, hi, ctrl, 0xf, 0xf, true);
    return __hiloint2double(hi, lo);
}
template <int Q>
__device__ __forceinline__ float row_bcast(float v)
{
    constexpr int ctrl = 0x150 + Q;
    const int b = __float_as_int(v);
    return __int_as_float(__builtin_amdgcn_update_dpp(b, b, ctrl, 0xf, 0xf, true));
}
template <int LANES, int Q, typename T>
__device__ __forceinline__ T group_bcast(T v)
{
    static_assert(LANES == 4 || LANES == 16, "groups of four or sixteen lanes");
    if constexpr (LANES == 4) return quad_bcast<Q>(v);
    else return row_bcast<Q>(v);
}

// Forward substitution on kLeaf unknowns of one right-hand side shared by
// LANES lanes (4 or 16): lane q of the group holds the unknowns LANES * r + q
// in x[r]; mb points at this lane's rows of column 0 of the triangle in LDS
// (column l, row LANES * r + q at mb[l * LD + LANES * r], reciprocals on
// the diagonal).  With more lanes a step has fewer multiply-adds per lane and
// comes closer to the bare chain finish -> broadcast -> multiply-add.
//
// Unrolled at compile time so that x and two columns of the triangle stay
// in registers; column l+1 is read while column l is applied.  The empty
// asm statements fix that order: without them the compiler either hoists
// every LDS read to the top or waits for each read right before its use.
template <typename T, int LANES, int LD = kLeaf>
__device__ __forceinline__ void substitute(T (&x)[kLeaf / LANES], const T *mb, const int q)
{
    constexpr int R = kLeaf / LANES;
    T mc[2][R];
    static_for<0, R>([&](auto rc) { mc[0][decltype(rc)::value] = mb[LANES * decltype(rc)::value]; });
    static_for<0, kLeaf>([&](auto lc) {
        constexpr int l = decltype(lc)::value;
        constexpr int p = l & 1, ro = l / LANES, qo = l % LANES;
        constexpr int ln = l + 1 < kLeaf ? l + 1 : l;
        asm volatile("" ::: "memory");
        static_for<(ln / LANES), R>([&](auto rc) {
            mc[1 - p][decltype(rc)::value] = mb[ln * LD + LANES * decltype(rc)::value];
        });
        // the owner of unknown l finishes it, everybody in the group receives it
        const T fin = x[ro] * mc[p][ro];
        x[ro] = (q == qo) ? fin : x[ro];
        const T xl = group_bcast<LANES, qo>(x[ro]);
        if constexpr (qo < LANES - 1) {
            const T upd = x[ro] - mc[p][ro] * xl;
            x[ro] = (q > qo) ? upd : x[ro];
        }
        static_for<ro + 1, R>([&](auto rc) {
            constexpr int r = decltype(rc)::value;
            x[r] -= mc[p][r] * xl;
        });
        static_for<ro, R>([&](auto rc) { pin(x[decltype(rc)::value]); });
    });
}

// The product x <- M x on the same layout (the diagonal itself on the diagonal
// of the triangle in LDS): columns applied from the last to the first so that
// every x_l is still the old value when it is used (x_i += M[i][l] x_l for
// i > l, x_l <- M[l][l] x_l).
template <typename T, int LANES, int LD = kLeaf>
__device__ __forceinline__ void multiply_leaf(T (&x)[kLeaf / LANES], const T *mb, const int q)
{
    constexpr int R = kLeaf / LANES;
    T mc[2][R];
    static_for<0, R>([&](auto rc) {
        mc[0][decltype(rc)::value] = mb[(kLeaf - 1) * LD + LANES * decltype(rc)::value];
    });
    static_for<0, kLeaf>([&](auto lc) {
        constexpr int l = kLeaf - 1 - decltype(lc)::value;
        constexpr int p = decltype(lc)::value & 1, ro = l / LANES, qo = l % LANES;
        constexpr int ln = l > 0 ? l - 1 : 0;
        asm volatile("" ::: "memory");
        static_for<(ln / LANES), R>([&](auto rc) {
            mc[1 - p][decltype(rc)::value] = mb[ln * LD + LANES * decltype(rc)::value];
        });
        const T xl = group_bcast<LANES, qo>(x[ro]);        // the old x_l
        const T own = mc[p][ro] * xl;
        const T upd = x[ro] + mc[p][ro] * xl;
        x[ro] = (q == qo) ? own : ((q > qo) ? upd : x[ro]);
        static_for<ro + 1, R>([&](auto rc) {
            constexpr int r = decltype(rc)::value;
            x[r] += mc[p][r] * xl;
        });
        static_for<ro, R>([&](auto rc) { pin(x[decltype(rc)::value]); });
    });
}

// Forward substitution x_l = d_l * (b_l - sum_{i<l} M[l][i] x_i) on kLeaf
// unknowns for kLeafVecs right-hand sides per workgroup.  Four lanes share a
// right-hand side: lane q of the four keeps the unknowns i = 4r + q in
// registers, so every step costs a quarter of the column's multiply-adds per
// lane plus one broadcast of the unknown that has just become final.  The
// triangle sits in LDS (reciprocal diagonal), the block of B passes through
// LDS on its way in and out so that global memory is read and written along
// whichever of its two directions is contiguous.  Blocks smaller than kLeaf
// are padded with the identity; backward solves run through the same code on
// reversed indices.  Only the triangle of A that BLAS declares as referenced
// is read.
//
// MULT = true is the triangular product on the same data layout: x <- M x,
// columns applied from the last to the first so that every x_l is still the
// old value when it is used (x_i += M[i][l] x_l for i > l, x_l <- M[l][l] x_l).
template <typename T, bool MULT>
__global__ __launch_bounds__(kLoadThreads) void trsm_leaf_kernel(LeafArgs<T> a)
{
    // Ms[l][i]: column l of M, entries i > l; Ms[l][l] holds the reciprocal of the diagonal (the diagonal itself
    // for the product)
    __shared__ T Ms[kLeaf][kLeaf];
    __shared__ T Xs[kLeafVecs][kLeaf + 1];      // Xs[v][i]: unknown i of right-hand side v
    const int tid = threadIdx.x;
    const int nb = a.nb;

    // all threads fetch the triangle, kPerThread independent loads each
    constexpr int kPerThread = kLeaf * kLeaf / kLoadThreads;
    T mv[kPerThread];
#pragma unroll
    for (int q = 0; q < kPerThread; ++q) {
        const int idx = tid + q * kLoadThreads;
        const int i = idx % kLeaf, l = idx / kLeaf;
        T v = (i == l) ? T(1) : T(0);
        if (i < nb && l < nb && (i > l || (i == l && !a.unit))) {
            const int ri = a.reversed ? nb - 1 - i : i;
            const int rl = a.reversed ? nb - 1 - l : l;
            v = a.A[ri * a.a_si + rl * a.a_sl];
        }
        mv[q] = v;
    }
    // ... and this workgroup's block of B, along its contiguous direction
    const int64_t v0 = (int64_t)blockIdx.x * kLeafVecs;
    const int nv = (int)((a.nvec - v0 < kLeafVecs) ? a.nvec - v0 : kLeafVecs);
    const bool i_fast = a.b_si <= a.b_sv;
    constexpr int kPerThreadB = kLeaf * kLeafVecs / kLoadThreads;
    T bv[kPerThreadB];
#pragma unroll
    for (int q = 0; q < kPerThreadB; ++q) {
        const int idx = tid + q * kLoadThreads;
        const int i = i_fast ? idx % kLeaf : idx / kLeafVecs, v = i_fast ? idx / kLeaf : idx % kLeafVecs;
        T val = T(0);
        if (i < nb && v < nv) {
            const int ri = a.reversed ? nb - 1 - i : i;
            val = a.B[ri * a.b_si + (v0 + v) * a.b_sv];
        }
        bv[q] = val;
    }
#pragma unroll
    for (int q = 0; q < kPerThread; ++q) {
        const int idx = tid + q * kLoadThreads;
        const int i = idx % kLeaf, l = idx / kLeaf;
        Ms[l][i] = (i == l && !MULT) ? T(1) / mv[q] : mv[q];
    }
#pragma unroll
    for (int q = 0; q < kPerThreadB; ++q) {
        const int idx = tid + q * kLoadThreads;
        const int i = i_fast ? idx % kLeaf : idx / kLeafVecs, v = i_fast ? idx / kLeaf : idx % kLeafVecs;
        Xs[v][i] = (a.alpha != T(1)) ? bv[q] * a.alpha : bv[q];
    }
    __syncthreads();

    constexpr int R = kLeaf / 4;          // unknowns per lane
    const int q = tid & 3, v = tid >> 2;
    T x[R];
#pragma unroll
    for (int r = 0; r < R; ++r) x[r] = Xs[v][4 * r + q];
    const T *mb = &Ms[0][q];              // this lane's rows of column l: mb[l * kLeaf + 4 r]

    if constexpr (!MULT) {
        substitute<T, 4>(x, mb, q);
    } else {
        multiply_leaf<T, 4>(x, mb, q);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) Xs[v][4 * r + q] = x[r];
    __syncthreads();
#pragma unroll
    for (int qq = 0; qq < kPerThreadB; ++qq) {
        const int idx = tid + qq * kLoadThreads;
        const int i = i_fast ? idx % kLeaf : idx / kLeafVecs, vv = i_fast ? idx / kLeaf : idx % kLeafVecs;
        if (i < nb && vv < nv) {
            const int ri = a.reversed ? nb - 1 - i : i;
            a.B[ri * a.b_si + (v0 + vv) * a.b_sv] = Xs[vv][i];
        }
    }
}

// ---------------------------------------------------------------------------
// A block of up to kBlock = 4 * kLeaf unknowns in one launch.  Right-hand
// sides do not depend on each other, so a workgroup that keeps its
// kBlockVecs right-hand sides in LDS can walk the whole block alone: solve
// leaf j by substitution (sixteen lanes per right-hand side, so that a step
// is little more than the chain finish -> broadcast -> multiply-add), then
// subtract leaf j's contribution from the leaves below it with 16x16x4 matrix
// instructions (one 16 x 16 tile of every leaf per wavefront; the operand
// from A goes from global memory straight into registers and is requested
// before the substitution starts, so that its latency is hidden).
// This replaces a chain of four leaf launches and three thin GEMM launches.
// MULT = true is the triangular product on the same plan: leaves from the
// last to the first, each one handing its old values to the leaves below it
// before it is multiplied by its own triangle.
typedef double trsm_d4 __attribute__((ext_vector_type(4)));
typedef float trsm_f4 __attribute__((ext_vector_type(4)));

template <typename T>
struct Mfma16;
template <>
struct Mfma16<double> {
    typedef trsm_d4 Acc;
    static __device__ __forceinline__ Acc run(double x, double y, Acc c)
    {
        return __builtin_amdgcn_mfma_f64_16x16x4f64(x, y, c, 0, 0, 0);
    }
    // row of the 16 x 16 result that register r of this lane holds (the column is lane % 16)
    static __device__ __forceinline__ int row(int r, int lane) { return 4 * r + (lane >> 4); }
};
template <>
struct Mfma16<float> {
    typedef trsm_f4 Acc;
    static __device__ __forceinline__ Acc run(float x, float y, Acc c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x4f32(x, y, c, 0, 0, 0);
    }
    static __device__ __forceinline__ int row(int r, int lane) { return 4 * (lane >> 4) + r; }
};

constexpr int kBlockSub = 4;                  // leaves per block
constexpr int kBlock = kBlockSub * kLeaf;     // unknowns per block
constexpr int kBlockVecs = 32;                // right-hand sides per workgroup
constexpr int kBlockLanes = 16;               // lanes that share a right-hand side in the leaves
constexpr int kBlockThreads = kBlockVecs * kBlockLanes;   // eight wavefronts
constexpr int kWideParts = 2;                 // parts of kBlock unknowns that one launch of the solve can take
std::atomic<int> g_wide_parts{kWideParts};    // the same as the solver uses it (1: one part per launch)

//
// PARTS > 1 (the solve only): up to PARTS such blocks ("parts") in one launch.
// What a finished part contributes to the parts after it -- (rows of the later
// part, columns of this one) of M times this part's solution -- is worked out
// by the same workgroup with matrix instructions and kept in registers until
// the later part's turn comes; this replaces a launch of the GEMM with k = 256
// and a second launch of this kernel.
//
// KFAST says along which of M's two directions memory is contiguous: along
// the rows' index i (false) or along the columns' index l (true), which is the
// k of the matrix instructions.  A slice of M for those instructions is 16
// rows by 64 columns, lane % 16 the row.  With KFAST false the 16 rows of a
// column are one 128-byte run, so lane / 16 + 4 kk is the column of register
// kk and every load instruction touches four such runs.  With KFAST true
// that assignment would touch 16 rows' lines for 32 bytes each, 16 times over;
// the instructions do not care in which order k runs as long as both operands
// agree, so there a lane takes four consecutive columns per load,
// 16 (kk / 4) + 4 (lane / 16) + kk % 4, and the other operand is read from
// LDS to match.
template <typename T, bool KFAST>
struct Slice {
    typedef T V4 __attribute__((ext_vector_type(4)));
    typedef V4 V4U __attribute__((aligned(sizeof(T))));
    // column of M (relative to the slice's first) that register kk of a lane in group g = lane / 16 holds,
    // in the order of the solve
    static __device__ __forceinline__ int column(int kk, int g)
    {
        return KFAST ? 16 * (kk >> 2) + 4 * g + (kk & 3) : 4 * kk + g;
    }
    // N registers of row `row` (index in memory order, i.e. after the reversal), columns from col0 (in the order of
    // the solve; the solve's column c sits at nb - 1 - c when reversed).  With KFAST and a reversed solve the four
    // registers of a load come out in the opposite order: register kk holds what column(kk ^ 3, g) says.
    template <int N>
    static __device__ __forceinline__ void load(T (&f)[N], const LeafArgs<T> &a, int row, bool live, int col0, int g)
    {
        if constexpr (KFAST) {
            const T *src = a.A + (int64_t)row * a.a_si;
#pragma unroll
            for (int p = 0; p < N / 4; ++p) {
                const int c = col0 + 16 * p + 4 * g;
                const int at = a.reversed ? a.nb - 1 - (c + 3) : c;
                V4 v = {0, 0, 0, 0};
                if (live) v = *reinterpret_cast<const V4U *>(src + at);
#pragma unroll
                for (int e = 0; e < 4; ++e) f[4 * p + e] = v[e];
            }
        } else {
            const int c = col0 + g;
            const T *src = a.A + (int64_t)row * a.a_si + (int64_t)(a.reversed ? a.nb - 1 - c : c) * a.a_sl;
            const int64_t col_step = (a.reversed ? -4 : 4) * a.a_sl;
#pragma unroll
            for (int kk = 0; kk < N; ++kk) f[kk] = live ? src[kk * col_step] : T(0);
        }
    }
};

constexpr int kTriLd = kLeaf + 1;             // leading dimension of the triangle in LDS: odd, so that it can be
                                              // written along either of its directions

template <typename T, bool MULT, int PARTS, bool KFAST>
__global__ __launch_bounds__(kBlockThreads) void trsm_block_kernel(LeafArgs<T> a)
{
    static_assert(PARTS >= 1 && (!MULT || PARTS == 1), "the product walks one part of kBlock unknowns");
    typedef Mfma16<T> MF;
    typedef typename MF::Acc Acc;
    typedef Slice<T, KFAST> SL;
    __shared__ T Ms[kLeaf][kTriLd];                 // as in the leaf kernel, for the leaf being worked on
    __shared__ T Xs[kBlockVecs][kBlock + 1];        // Xs[v][i]: unknown i (of the part at hand) of right-hand side v
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nb = a.nb;
    const int nsub = (nb + kLeaf - 1) / kLeaf;
    const int parts = (nsub + kBlockSub - 1) / kBlockSub;
    const int64_t v0 = (int64_t)blockIdx.x * kBlockVecs;
    const int nv = (int)((a.nvec - v0 < kBlockVecs) ? a.nvec - v0 : kBlockVecs);
    const bool i_fast = a.b_si <= a.b_sv;
    auto rev = [&](int i) { return a.reversed ? nb - 1 - i : i; };

    // element (i, l) of leaf j's triangle as the leaf code wants it (identity outside the block)
    constexpr int kTriPerThread = kLeaf * kLeaf / kBlockThreads;
    // Thread t takes, along the direction that is contiguous in memory, element t % kLeaf, and across it the
    // elements t / kLeaf + q * (kBlockThreads / kLeaf).
    auto tri_place = [&](int q, int &i, int &l) {
        const int fast = tid % kLeaf, slow = tid / kLeaf + q * (kBlockThreads / kLeaf);
        i = KFAST ? slow : fast;
        l = KFAST ? fast : slow;
    };
    auto load_triangle = [&](int j, T (&mv)[kTriPerThread]) {
#pragma unroll
        for (int q = 0; q < kTriPerThread; ++q) {
            int i, l;
            tri_place(q, i, l);
            const int gi = j * kLeaf + i, gl = j * kLeaf + l;
            T v = (i == l) ? T(1) : T(0);
            if (gi < nb && gl < nb && (i > l || (i == l && !a.unit)))
                v = a.A[(int64_t)rev(gi) * a.a_si + (int64_t)rev(gl) * a.a_sl];
            mv[q] = v;
        }
    };
    // the solve walks the leaves downwards, the product upwards (every leaf
    // must still hold its old values when the leaves below it take their share)
    T mv[kTriPerThread];
    load_triangle(MULT ? nsub - 1 : 0, mv);

    // A part of this workgroup's block of B: leaf by leaf, along its contiguous direction; all
    // loads are issued before the first value is used.  Thread t moves, of leaf s, the elements
    // t + q * kBlockThreads of the leaf's kLeaf x kBlockVecs values.
    constexpr int kPerThreadB = kLeaf * kBlockVecs / kBlockThreads;
    int tid_b = tid;     // re-made opaque after every leaf loop, so that addresses are worked out where they are used
    auto b_place = [&](int s, int q, int &i, int &v) {
        const int idx = tid_b + q * kBlockThreads;
        i = s * kLeaf + (i_fast ? idx % kLeaf : idx / kBlockVecs);
        v = i_fast ? idx / kLeaf : idx % kBlockVecs;
    };
    T bv[kBlockSub][kPerThreadB];
    auto fetch_part = [&](int h) {
#pragma unroll
        for (int s = 0; s < kBlockSub; ++s) {
#pragma unroll
            for (int q = 0; q < kPerThreadB; ++q) {
                int i, v;
                b_place(s, q, i, v);
                T val = T(0);
                if (h * kBlock + i < nb && v < nv) val = a.B[rev(h * kBlock + i) * a.b_si + (v0 + v) * a.b_sv];
                bv[s][q] = (a.alpha != T(1)) ? val * a.alpha : val;
            }
        }
    };
    fetch_part(0);

    // What the parts already solved contribute to the parts after them, kept in
    // registers until a part's turn comes: later[d] belongs to the d-th part
    // after the one at hand.  Of every part a wavefront holds the blocks of 16
    // rows `wave` and `wave + 8` for both groups of 16 right-hand sides.
    constexpr int kLater = PARTS > 1 ? PARTS - 1 : 1;
    Acc later[kLater][2][2];
    if constexpr (PARTS > 1) {
#pragma unroll
        for (int d = 0; d < kLater; ++d)
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int u = 0; u < 2; ++u) later[d][t][u] = Acc{0, 0, 0, 0};
    }

    constexpr int R = kLeaf / kBlockLanes;
    constexpr int kMaxPairs = kBlockSub - 1;     // leaves below the current one: tiles per wavefront and step
    const int mt = wave & 3, nt = wave >> 2;     // this wavefront's 16 rows of every leaf, its 16 right-hand sides
    const bool flipped = KFAST && a.reversed;    // Slice::load: the registers of a slice of M run against those of X

    static_for<0, PARTS>([&](auto hc) {
        constexpr int h = decltype(hc)::value;
        if (h >= parts) return;
        const int nl = (nsub - h * kBlockSub < kBlockSub) ? nsub - h * kBlockSub : kBlockSub;   // leaves of this part

        // alpha * B of this part into LDS, less what the parts before it contribute
        if constexpr (h > 0) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    T *dst = &Xs[u * 16 + (lane & 15)][(wave + 8 * t) * 16];
#pragma unroll
                    for (int r = 0; r < 4; ++r) dst[MF::row(r, lane)] = -later[0][t][u][r];
                }
            }
            __syncthreads();
#pragma unroll
            for (int s = 0; s < kBlockSub; ++s) {
#pragma unroll
                for (int q = 0; q < kPerThreadB; ++q) {
                    int i, v;
                    b_place(s, q, i, v);
                    Xs[v][i] += bv[s][q];
                }
            }
            // the parts after this one move up
#pragma unroll
            for (int d = 0; d + 1 < kLater; ++d)
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int u = 0; u < 2; ++u) later[d][t][u] = later[d + 1][t][u];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int u = 0; u < 2; ++u) later[kLater - 1][t][u] = Acc{0, 0, 0, 0};
        } else {
#pragma unroll
            for (int s = 0; s < kBlockSub; ++s) {
                if (s < nl) {
#pragma unroll
                    for (int q = 0; q < kPerThreadB; ++q) {
                        int i, v;
                        b_place(s, q, i, v);
                        Xs[v][i] = bv[s][q];
                    }
                }
            }
        }

        for (int step = 0; step < nl; ++step) {
            const int jl = MULT ? nl - 1 - step : step;      // leaf within the part
            const int j = h * kBlockSub + jl;                 // and within the block
            {
                // a thread holds at most one element of the diagonal: one division
                T dg = T(1);
#pragma unroll
                for (int q = 0; q < kTriPerThread; ++q) {
                    int i, l;
                    tri_place(q, i, l);
                    if (i == l) dg = mv[q];
                }
                if constexpr (!MULT) dg = T(1) / dg;
#pragma unroll
                for (int q = 0; q < kTriPerThread; ++q) {
                    int i, l;
                    tri_place(q, i, l);
                    Ms[l][i] = (i == l) ? dg : mv[q];
                }
            }
            // leaf j as the second operand of the matrix instructions: element
            // (k as Slice says, vector 16 nt + lane % 16); the solve reads it
            // once leaf j is final, the product before leaf j changes
            T bf[kLeaf / 4];
            auto read_leaf = [&]() {
#pragma unroll
                for (int kk = 0; kk < kLeaf / 4; ++kk)
                    bf[kk] = Xs[nt * 16 + (lane & 15)][jl * kLeaf + SL::column(kk, lane >> 4)];
            };
            if constexpr (MULT) read_leaf();
            __syncthreads();

            // Requests that the leaf code below does not wait for: the next
            // leaf's triangle, and the slices of A that couple leaf j to the
            // leaves of the part below it: of every such leaf this wavefront's 16 rows; lane
            // holds element (row lane % 16, column 4 kk + lane / 16), kk = 0 .. 15.
            if (step + 1 < nl) load_triangle(MULT ? j - 1 : j + 1, mv);
            const int npairs = nl - 1 - jl;          // per wavefront
            T af[kMaxPairs][kLeaf / 4];
#pragma unroll
            for (int pp = 0; pp < kMaxPairs; ++pp) {
                if (pp < npairs) {
                    const int gi = (j + 1 + pp) * kLeaf + mt * 16 + (lane & 15);
                    SL::load(af[pp], a, rev(gi < nb ? gi : 0), gi < nb, j * kLeaf, lane >> 4);
                }
            }

            {
                const int q = tid % kBlockLanes, v = tid / kBlockLanes;
                T x[R];
                T *xv = &Xs[v][jl * kLeaf + q];
#pragma unroll
                for (int r = 0; r < R; ++r) x[r] = xv[kBlockLanes * r];
                if constexpr (MULT) multiply_leaf<T, kBlockLanes, kTriLd>(x, &Ms[0][q], q);
                else substitute<T, kBlockLanes, kTriLd>(x, &Ms[0][q], q);
#pragma unroll
                for (int r = 0; r < R; ++r) xv[kBlockLanes * r] = x[r];
            }
            if constexpr (!MULT) {
                __syncthreads();
                if (npairs > 0) read_leaf();
            }
#pragma unroll
            for (int pp = 0; pp < kMaxPairs; ++pp) {
                if (pp < npairs) {
                    Acc acc = {0, 0, 0, 0};
                    if (flipped) {
#pragma unroll
                        for (int kk = 0; kk < kLeaf / 4; ++kk) acc = MF::run(af[pp][kk], bf[kk ^ 3], acc);
                    } else {
#pragma unroll
                        for (int kk = 0; kk < kLeaf / 4; ++kk) acc = MF::run(af[pp][kk], bf[kk], acc);
                    }
                    T *dst = &Xs[nt * 16 + (lane & 15)][(jl + 1 + pp) * kLeaf + mt * 16];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if constexpr (MULT) dst[MF::row(r, lane)] += acc[r];
                        else dst[MF::row(r, lane)] -= acc[r];
                    }
                }
            }
            // The solve's next step separates these writes from its reads with its
            // first barrier; the product's next step reads leaf j - 1 at once and
            // overwrites the triangle that the leaf code above may still be using.
            if constexpr (MULT) __syncthreads();
        }
        __syncthreads();
        asm volatile("" : "+v"(tid_b));

        if constexpr (h + 1 < PARTS) {
            if (h + 1 < parts) {
                // The next part's right-hand sides are requested now and arrive during the
                // products.  For every later part g: (rows of part g, columns of this part)
                // of M times this part's solution, 64 columns (one leaf) at a time; the
                // slices of M go from memory straight into registers, three slices ahead of the
                // matrix instructions that use them.
                fetch_part(h + 1);
                constexpr int kLive = PARTS - 1 - h;          // parts after this one, at most
                constexpr int kCols = 16;                     // columns of M per slice
                constexpr int kBufs = 4;                      // slices in registers: kBufs - 1 on their way
                constexpr int kPerLeaf = kLeaf / kCols;
                constexpr int kSlices = kBlockSub * kPerLeaf * kLive * 2;
                // slice f, from the slowest index to the fastest: leaf of this part, later part,
                // row block wave + 8 t, run of kCols columns of the leaf
                T fr[kBufs][kCols / 4];
                auto fetch_slice = [&](int f, T (&dst)[kCols / 4]) {
                    const int c = f % kPerLeaf, t = (f / kPerLeaf) % 2, d = (f / (2 * kPerLeaf)) % kLive;
                    const int jl = f / (2 * kPerLeaf * kLive);
                    const int gi = (h + 1 + d) * kBlock + (wave + 8 * t) * 16 + (lane & 15);
                    SL::load(dst, a, rev(gi < nb ? gi : 0), gi < nb, h * kBlock + jl * kLeaf + c * kCols, lane >> 4);
                };
                static_for<0, kBufs - 1>([&](auto fc) { fetch_slice(decltype(fc)::value, fr[decltype(fc)::value]); });
                T xf[2][kLeaf / 4];
                static_for<0, kSlices>([&](auto fc) {
                    constexpr int f = decltype(fc)::value;
                    constexpr int c = f % kPerLeaf, t = (f / kPerLeaf) % 2, d = (f / (2 * kPerLeaf)) % kLive;
                    constexpr int jl = f / (2 * kPerLeaf * kLive);
                    if constexpr (f % (2 * kPerLeaf * kLive) == 0) {
#pragma unroll
                        for (int u = 0; u < 2; ++u)
#pragma unroll
                            for (int kk = 0; kk < kLeaf / 4; ++kk)
                                xf[u][kk] = Xs[u * 16 + (lane & 15)][jl * kLeaf + SL::column(kk, lane >> 4)];
                    }
                    if constexpr (f + kBufs - 1 < kSlices) fetch_slice(f + kBufs - 1, fr[(f + kBufs - 1) % kBufs]);
                    if (h + 1 + d < parts) {
                        if (flipped) {
#pragma unroll
                            for (int kk = 0; kk < kCols / 4; ++kk) {
                                later[d][t][0] = MF::run(fr[f % kBufs][kk], xf[0][c * (kCols / 4) + (kk ^ 3)], later[d][t][0]);
                                later[d][t][1] = MF::run(fr[f % kBufs][kk], xf[1][c * (kCols / 4) + (kk ^ 3)], later[d][t][1]);
                            }
                        } else {
#pragma unroll
                            for (int kk = 0; kk < kCols / 4; ++kk) {
                                later[d][t][0] = MF::run(fr[f % kBufs][kk], xf[0][c * (kCols / 4) + kk], later[d][t][0]);
                                later[d][t][1] = MF::run(fr[f % kBufs][kk], xf[1][c * (kCols / 4) + kk], later[d][t][1]);
                            }
                        }
                    }
                });
            }
        }

        for (int s = 0; s < nl; ++s) {
#pragma unroll
            for (int q = 0; q < kPerThreadB; ++q) {
                int i, v;
                b_place(s, q, i, v);
                if (h * kBlock + i < nb && v < nv) a.B[rev(h * kBlock + i) * a.b_si + (v0 + v) * a.b_sv] = Xs[v][i];
            }
        }
        if constexpr (h + 1 < PARTS) {
            if (h + 1 < parts) {
                load_triangle((h + 1) * kBlockSub, mv);
                __syncthreads();
            }
        }
    });
}

// The eight BLAS cases in one description.  The unknowns are indexed along
// the triangular dimension (rows of B for side = left, columns for right);
// "forward" means unknown i depends on the unknowns before it.
template <typename T, bool MULT = false>
struct Solve {
    bool right, trans, unit, forward;
    int nrhs;               // extent of B across the triangular dimension
    const T *A;
    int ldA;
    T *B;
    int ldB;
    hipStream_t stream;

    // op(A)[i, l] for i, l along the triangular dimension
    const T *a_at(int i, int l) const
    {
        return trans ? A + (int64_t)l + (int64_t)i * ldA : A + (int64_t)i + (int64_t)l * ldA;
    }
    // first element of the block of B whose unknowns start at i
    T *b_at(int i) const { return right ? B + (int64_t)i * ldB : B + i; }

    int leaf(int at, int nb, T alpha) const
    {
        LeafArgs<T> a;
        a.A = a_at(at, at);
        // left:  M = op(A);    M[i][l] = op(A)[i, l]
        // right: M = op(A)^T;  M[i][l] = op(A)[l, i]
        int64_t si = trans ? ldA : 1, sl = trans ? 1 : ldA;
        if (right) std::swap(si, sl);
        a.a_si = si;
        a.a_sl = sl;
        a.B = b_at(at);
        a.b_si = right ? ldB : 1;
        a.b_sv = right ? 1 : ldB;
        a.nb = nb;
        a.nvec = nrhs;
        a.reversed = forward ? 0 : 1;
        a.unit = unit ? 1 : 0;
        a.alpha = alpha;
        const int blocks = (nrhs + kLeafVecs - 1) / kLeafVecs;
        hipLaunchKernelGGL((trsm_leaf_kernel<T, MULT>), dim3(blocks), dim3(kLoadThreads), 0, stream, a);
        HIP_TRY(hipGetLastError());
        return ULMBLAS_GPU_OK;
    }

    // leaf() for up to kBlock unknowns (the solve: up to kWideParts * kBlock)
    int block(int at, int nb, T alpha) const
    {
        LeafArgs<T> a;
        a.A = a_at(at, at);
        int64_t si = trans ? ldA : 1, sl = trans ? 1 : ldA;
        if (right) std::swap(si, sl);
        a.a_si = si;
        a.a_sl = sl;
        a.B = b_at(at);
        a.b_si = right ? ldB : 1;
        a.b_sv = right ? 1 : ldB;
        a.nb = nb;
        a.nvec = nrhs;
        a.reversed = forward ? 0 : 1;
        a.unit = unit ? 1 : 0;
        a.alpha = alpha;
        const int blocks = (nrhs + kBlockVecs - 1) / kBlockVecs;
        const bool kfast = a.a_sl == 1;       // M contiguous along its columns: see Slice
        bool wide = false;
        if constexpr (!MULT) wide = nb > kBlock;
        auto kernel = trsm_block_kernel<T, MULT, 1, false>;
        if (!wide) {
            if (kfast) kernel = trsm_block_kernel<T, MULT, 1, true>;
        } else if constexpr (!MULT) {
            kernel = kfast ? trsm_block_kernel<T, MULT, kWideParts, true> : trsm_block_kernel<T, MULT, kWideParts, false>;
        }
        hipLaunchKernelGGL(kernel, dim3(blocks), dim3(kBlockThreads), 0, stream, a);
        HIP_TRY(hipGetLastError());
        return ULMBLAS_GPU_OK;
    }

    // B[dst block] <- scale * B[dst block] + factor * (coupling block of op(A)) * B[src block]
    int update(int dst, int ndst, int src, int nsrc, T factor, T scale) const
    {
        if (!right) {
            // rows dst.. of B += factor * op(A)[dst.., src..] * rows src.. of B
            const T *blk = trans ? A + src + (int64_t)dst * ldA : A + dst + (int64_t)src * ldA;
            return gemm_device<T>(trans, false, ndst, nrhs, nsrc, factor, blk, ldA, b_at(src), ldB, scale,
                                  b_at(dst), ldB, stream);
        }
        // columns dst.. of B += factor * columns src.. of B * op(A)[src.., dst..]
        const T *blk = trans ? A + dst + (int64_t)src * ldA : A + src + (int64_t)dst * ldA;
        return gemm_device<T>(false, trans, nrhs, ndst, nsrc, factor, b_at(src), ldB, blk, ldA, scale, b_at(dst),
                              ldB, stream);
    }

    // The product B <- alpha * M * B on the unknowns [at, at + len), M = op(A)
    // (or its transpose for the right side) lower triangular when `forward`:
    // the half that depends on the other one goes first, then receives the
    // other half's (still unchanged) contribution, then the other half follows.
    int multiply(int at, int len, T alpha) const
    {
        if (len <= kLeaf) return leaf(at, len, alpha);
        if (len <= kBlock) return block(at, len, alpha);
        const int half = ((len / 2 + kBlock - 1) / kBlock) * kBlock;
        int rc;
        if (forward) {      // [M11 0; M21 M22]: bottom = M22 bottom + M21 top, then top = M11 top
            if ((rc = multiply(at + half, len - half, alpha))) return rc;
            if ((rc = update(at + half, len - half, at, half, alpha, T(1)))) return rc;
            return multiply(at, half, alpha);
        }
        const int low = len - half;     // [M11 M12; 0 M22]: top = M11 top + M12 bottom, then bottom = M22 bottom
        if ((rc = multiply(at, low, alpha))) return rc;
        if ((rc = update(at, low, at + low, half, alpha, T(1)))) return rc;
        return multiply(at + low, half, alpha);
    }

    // Solve the unknowns [at, at + len).  Their right-hand sides still carry
    // the factor `alpha` to be applied (the caller's alpha on first touch,
    // 1 once an update has folded it in).
    int run(int at, int len, T alpha) const
    {
        if (len <= kLeaf) return leaf(at, len, alpha);
        if (len <= g_wide_parts.load() * kBlock) return block(at, len, alpha);
        const int half = ((len / 2 + kBlock - 1) / kBlock) * kBlock;
        int rc;
        if (forward) {
            if ((rc = run(at, half, alpha))) return rc;
            if ((rc = update(at + half, len - half, at, half, T(-1), alpha))) return rc;
            return run(at + half, len - half, T(1));
        }
        const int low = len - half;    // the trailing `half` unknowns are solved first
        if ((rc = run(at + low, half, alpha))) return rc;
        if ((rc = update(at, low, at + low, half, T(-1), alpha))) return rc;
        return run(at, low, T(1));
    }
};

int trsm_set_parts(int parts)
{
    if (parts < 1 || parts > kWideParts) return ULMBLAS_GPU_BAD_ARGUMENT;
    g_wide_parts.store(parts);
    return ULMBLAS_GPU_OK;
}

template <typename T>
int trsm_device(bool right, bool lower, bool trans, bool unit, int m, int n, T alpha, const T *dA, int ldA, T *dB,
                int ldB, hipStream_t stream)
{
    const int ka = right ? n : m;
    if (m < 0 || n < 0 || ldA < std::max(1, ka) || ldB < std::max(1, m)) {
        g_last_error = "invalid size or leading dimension";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    if (m == 0 || n == 0) return ULMBLAS_GPU_OK;
    if (!dB || (alpha != T(0) && !dA)) {
        g_last_error = "null operand";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    // ulmblas/level3/trlsm.tcc:46-49: alpha == 0 stores zeros, A is not read
    if (alpha == T(0)) return launch_scale<T>(m, n, T(0), dB, ldB, stream);

    Solve<T> s;
    s.right = right;
    s.trans = trans;
    s.unit = unit;
    // op(A) lower triangular: left solves run forward, right solves backward
    const bool op_lower = (lower != trans);
    s.forward = right ? !op_lower : op_lower;
    s.nrhs = right ? m : n;
    s.A = dA;
    s.ldA = ldA;
    s.B = dB;
    s.ldB = ldB;
    s.stream = stream;
    return s.run(0, ka, alpha);
}

// B <- alpha*op(A)*B (left) or alpha*B*op(A) (right), A triangular: the
// operation of ulmBLAS::trlmm / trumm (ulmblas/level3/trlmm.tcc:16-88), same
// recursive splitting, leaves multiplied in registers.
template <typename T>
int trmm_device(bool right, bool lower, bool trans, bool unit, int m, int n, T alpha, const T *dA, int ldA, T *dB,
                int ldB, hipStream_t stream)
{
    const int ka = right ? n : m;
    if (m < 0 || n < 0 || ldA < std::max(1, ka) || ldB < std::max(1, m)) {
        g_last_error = "invalid size or leading dimension";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    if (m == 0 || n == 0) return ULMBLAS_GPU_OK;
    if (!dB || (alpha != T(0) && !dA)) {
        g_last_error = "null operand";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    // ulmblas/level3/trlmm.tcc:45-48
    if (alpha == T(0)) return launch_scale<T>(m, n, T(0), dB, ldB, stream);
    Solve<T, true> s;
    s.right = right;
    s.trans = trans;
    s.unit = unit;
    const bool op_lower = (lower != trans);
    s.forward = right ? !op_lower : op_lower;
    s.nrhs = right ? m : n;
    s.A = dA;
    s.ldA = ldA;
    s.B = dB;
    s.ldB = ldB;
    s.stream = stream;
    return s.multiply(0, ka, alpha);
}

// Host-pointer path: A's ka x ka window and B go up, the solve (or, with
// `multiply`, the product) runs, B comes back.
template <typename T>
int trsm_host(bool right, bool lower, bool trans, bool unit, int m, int n, T alpha, const T *A, int ldA, T *B,
              int ldB, bool multiply = false)
{
    if (m <= 0 || n <= 0) return ULMBLAS_GPU_OK;
    return with_context([&](HostContext &c) -> int {
    int rc = c.ensure_stream();
    if (rc) return rc;
    const int ka = right ? n : m;
    if ((rc = c.reserve(2, (size_t)m * n * sizeof(T)))) return rc;
    T *dB = static_cast<T *>(c.buf[2]);
    T *dA = nullptr;
    const size_t bytes = ((size_t)ka * ka + 2 * (size_t)m * n) * sizeof(T);
    if (alpha != T(0) && streams_transfers(c, bytes, (size_t)std::max(ka, m) * sizeof(T))) {
        // Right-hand sides do not depend on each other: A goes up, then B travels in panels of
        // right-hand sides (columns of B for the left side; rows for the right side, each panel
        // a compact matrix of its own on the device), every panel up, solved and on its way back
        // while its neighbours are at another of the three steps.
        if ((rc = c.reserve(0, (size_t)ka * ka * sizeof(T)))) return rc;
        dA = static_cast<T *>(c.buf[0]);
        const int nrhs = right ? m : n, other = right ? n : m;
        // The blocks on the diagonal take as long for 2048 right-hand sides as for 32 (one workgroup
        // per 32, bound by the chain of substitutions), so panels are wide: a few of them already hide
        // most of the transfers (8192 x 8192: 16 panels 43 ms, 4 panels 27 ms on paper).
        int panels = (int)std::min<long>(8, std::max<long>(1, nrhs / 2048));
        const int per = ((nrhs + panels - 1) / panels + 255) / 256 * 256;
        panels = (nrhs + per - 1) / per;
        if ((rc = c.ensure_events(2 * (size_t)panels))) return rc;
        Pipeline<T> pipe(c);
        pipe.set_free_out(c.out_ring.count());
        if ((rc = pipe.upload(A, ldA, dA, ka, ka, ka))) return rc;
        for (int p = 0; p < panels; ++p) {
            const int r0 = p * per, nr = std::min(per, nrhs - r0);
            T *dBp = dB + (size_t)r0 * other;           // left: m x nr at pitch m; right: nr x n at pitch nr
            T *Bp = right ? B + r0 : B + (size_t)r0 * ldB;
            const int pm = right ? nr : m, pn = right ? n : nr;
            if ((rc = pipe.upload(Bp, ldB, dBp, pm, pm, pn))) return rc;
            hipEvent_t uploaded = c.events[2 * p], solved = c.events[2 * p + 1];
            HIP_TRY(hipEventRecord(uploaded, c.h2d));
            HIP_TRY(hipStreamWaitEvent(c.stream, uploaded, 0));
            rc = multiply ? trmm_device<T>(right, lower, trans, unit, pm, pn, alpha, dA, ka, dBp, pm, c.stream)
                          : trsm_device<T>(right, lower, trans, unit, pm, pn, alpha, dA, ka, dBp, pm, c.stream);
            if (rc) return rc;
            HIP_TRY(hipEventRecord(solved, c.stream));
            pipe.want_download(dBp, Bp, ldB, pm, pn, solved);
            if ((rc = pipe.pump(false))) return rc;
        }
        if ((rc = pipe.pump(true))) return rc;
        HIP_TRY(hipStreamSynchronize(c.d2h));
        HIP_TRY(hipStreamSynchronize(c.h2d));
        HIP_TRY(hipStreamSynchronize(c.stream));
        return ULMBLAS_GPU_OK;
    }
    if (alpha != T(0)) {
        if ((rc = c.reserve(0, (size_t)ka * ka * sizeof(T)))) return rc;
        dA = static_cast<T *>(c.buf[0]);
        if ((rc = copy_window<T>(dA, (size_t)ka * sizeof(T), A, (size_t)ldA * sizeof(T), ka, ka,
                                 hipMemcpyHostToDevice, c.stream))) return rc;
        if ((rc = copy_window<T>(dB, (size_t)m * sizeof(T), B, (size_t)ldB * sizeof(T), m, n,
                                 hipMemcpyHostToDevice, c.stream))) return rc;
    }
    rc = multiply ? trmm_device<T>(right, lower, trans, unit, m, n, alpha, dA, ka, dB, m, c.stream)
                  : trsm_device<T>(right, lower, trans, unit, m, n, alpha, dA, ka, dB, m, c.stream);
    if (rc) return rc;
    if ((rc = copy_window<T>(B, (size_t)ldB * sizeof(T), dB, (size_t)m * sizeof(T), m, n, hipMemcpyDeviceToHost,
                             c.stream))) return rc;
    HIP_TRY(hipStreamSynchronize(c.stream));
    return ULMBLAS_GPU_OK;
    });
}

template <typename T>
void trsm_host_report(const char *rout, bool right, bool lower, bool trans, bool unit, int m, int n, T alpha,
                      const T *A, int ldA, T *B, int ldB, bool multiply = false)
{
    const int rc = trsm_host<T>(right, lower, trans, unit, m, n, alpha, A, ldA, B, ldB, multiply);
    report_host_status(rout, rc, nullptr);
}

// interfaces/blas/F77/trsm.cc:154-174
int f77_trsm_info(const char *side_, const char *upLo_, const char *transA_, const char *diag_, int m, int n,
                  int ldA, int ldB)
{
    const int sd = toupper((unsigned char)*side_), ul = toupper((unsigned char)*upLo_);
    const int ta = toupper((unsigned char)*transA_), dg = toupper((unsigned char)*diag_);
    const int numRowsA = (sd == 'L') ? m : n;
    if (sd != 'L' && sd != 'R') return 1;
    if (ul != 'L' && ul != 'U') return 2;
    if (ta != 'N' && ta != 'T' && ta != 'C' && ta != 'R') return 3;
    if (dg != 'U' && dg != 'N') return 4;
    if (m < 0) return 5;
    if (n < 0) return 6;
    if (ldA < std::max(1, numRowsA)) return 9;
    if (ldB < std::max(1, m)) return 11;
    return 0;
}

// interfaces/blas/C/trsm.cc:400-446
int cblas_trsm_info(int order, int side, int upLo, int transA, int diag, int m, int n, int ldA, int ldB)
{
    const int numRowsA = (side == CblasLeft) ? m : n;
    if (order != CblasColMajor && order != CblasRowMajor) return 1;
    if (side != CblasLeft && side != CblasRight) return 2;
    if (upLo != CblasLower && upLo != CblasUpper) return 3;
    if (transA != CblasNoTrans && transA != CblasTrans && transA != AtlasConj && transA != CblasConjTrans) return 4;
    if (diag != CblasUnit && diag != CblasNonUnit) return 5;
    if (order == CblasColMajor) {
        if (m < 0) return 6;
        if (n < 0) return 7;
        if (ldA < std::max(1, numRowsA)) return 10;
        if (ldB < std::max(1, m)) return 12;
    } else {
        if (n < 0) return 6;
        if (m < 0) return 7;
        if (ldA < std::max(1, numRowsA)) return 10;
        if (ldB < std::max(1, n)) return 12;
    }
    return 0;
}

// The triangular product takes the same arguments with the same checks
// (interfaces/blas/F77/trmm.cc:45-64, interfaces/blas/C/trmm.cc:402-437) and
// the same dispatch (F77/trmm.cc:176-229), so `multiply` is the only difference.
template <typename T>
void f77_trsm(const char *name6, const char *rout, const char *side, const char *upLo, const char *transA,
              const char *diag, int m, int n, T alpha, const T *A, int ldA, T *B, int ldB, bool multiply = false)
{
    int info = f77_trsm_info(side, upLo, transA, diag, m, n, ldA, ldB);
    if (info != 0) {
        xerbla_(name6, &info);
        return;
    }
    const int ta = toupper((unsigned char)*transA);
    trsm_host_report<T>(rout, toupper((unsigned char)*side) == 'R', toupper((unsigned char)*upLo) == 'L',
                        ta == 'T' || ta == 'C', toupper((unsigned char)*diag) == 'U', m, n, alpha, A, ldA, B, ldB,
                        multiply);
}

// interfaces/blas/C/trsm.cc:85-153 (ULMBLAS(dtrsm)): no checks; anything but
// CblasLeft is the right side, anything but CblasLower the upper triangle.
template <typename T>
void ulm_trsm(const char *rout, int side, int upLo, int transA, int diag, int m, int n, T alpha, const T *A,
              int ldA, T *B, int ldB, bool multiply = false)
{
    trsm_host_report<T>(rout, side != CblasLeft, upLo == CblasLower,
                        transA == CblasTrans || transA == CblasConjTrans, diag == CblasUnit, m, n, alpha, A, ldA, B,
                        ldB, multiply);
}

template <typename T>
void cblas_trsm(const char *rout, int order, int side, int upLo, int transA, int diag, int m, int n, T alpha,
                const T *A, int ldA, T *B, int ldB, bool multiply = false)
{
    int info = cblas_trsm_info(order, side, upLo, transA, diag, m, n, ldA, ldB);
    if (info != 0) {
        cblas_xerbla(info, rout, "");
        return;
    }
    if (order == CblasColMajor) {
        ulm_trsm<T>(rout, side, upLo, transA, diag, m, n, alpha, A, ldA, B, ldB, multiply);
    } else {   // interfaces/blas/C/trsm.cc:454-458
        side = (side == CblasLeft) ? CblasRight : CblasLeft;
        upLo = (upLo == CblasUpper) ? CblasLower : CblasUpper;
        ulm_trsm<T>(rout, side, upLo, transA, diag, n, m, alpha, A, ldA, B, ldB, multiply);
    }
}

template int trmm_device<double>(bool, bool, bool, bool, int, int, double, const double *, int, double *, int,
                                 hipStream_t);
template int trmm_device<float>(bool, bool, bool, bool, int, int, float, const float *, int, float *, int,
                                hipStream_t);
template int trsm_device<double>(bool, bool, bool, bool, int, int, double, const double *, int, double *, int,
                                 hipStream_t);
template int trsm_device<float>(bool, bool, bool, bool, int, int, float, const float *, int, float *, int,
                                hipStream_t);

}  // namespace ulmgpu

extern "C" {

void dtrsm_(const char *side, const char *upLo, const char *transA, const char *diag, const int *m, const int *n,
            const double *alpha, const double *A, const int *ldA, double *B, const int *ldB)
{
    f77_trsm<double>("DTRSM ", "dtrsm_", side, upLo, transA, diag, *m, *n, *alpha, A, *ldA, B, *ldB);
}

void strsm_(const char *side, const char *upLo, const char *transA, const char *diag, const int *m, const int *n,
            const float *alpha, const float *A, const int *ldA, float *B, const int *ldB)
{
    f77_trsm<float>("STRSM ", "strsm_", side, upLo, transA, diag, *m, *n, *alpha, A, *ldA, B, *ldB);
}

void cblas_dtrsm(enum CBLAS_ORDER order, enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE transA,
                 enum CBLAS_DIAG diag, int m, int n, double alpha, const double *A, int ldA, double *B, int ldB)
{
    cblas_trsm<double>("cblas_dtrsm", order, side, upLo, transA, diag, m, n, alpha, A, ldA, B, ldB);
}

void cblas_strsm(enum CBLAS_ORDER order, enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE transA,
                 enum CBLAS_DIAG diag, int m, int n, float alpha, const float *A, int ldA, float *B, int ldB)
{
    cblas_trsm<float>("cblas_strsm", order, side, upLo, transA, diag, m, n, alpha, A, ldA, B, ldB);
}

void ulmblas_dtrsm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE transA, enum CBLAS_DIAG diag,
                   int m, int n, double alpha, const double *A, int ldA, double *B, int ldB)
{
    ulm_trsm<double>("ulmblas_dtrsm", side, upLo, transA, diag, m, n, alpha, A, ldA, B, ldB);
}

void ulmblas_strsm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE transA, enum CBLAS_DIAG diag,
                   int m, int n, float alpha, const float *A, int ldA, float *B, int ldB)
{
    ulm_trsm<float>("ulmblas_strsm", side, upLo, transA, diag, m, n, alpha, A, ldA, B, ldB);
}

void ATL_dtrsm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE transA, enum CBLAS_DIAG diag, int m,
               int n, double alpha, const double *A, int ldA, double *B, int ldB)
{
    ulmblas_dtrsm(side, upLo, transA, diag, m, n, alpha, A, ldA, B, ldB);
}

void ATL_strsm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE transA, enum CBLAS_DIAG diag, int m,
               int n, float alpha, const float *A, int ldA, float *B, int ldB)
{
    ulmblas_strsm(side, upLo, transA, diag, m, n, alpha, A, ldA, B, ldB);
}

#define ULM_TRMM_ENTRY_POINTS(P, T, NAME6)                                                                             \
    void P##trmm_(const char *side, const char *upLo, const char *transA, const char *diag, const int *m,              \
                  const int *n, const T *alpha, const T *A, const int *ldA, T *B, const int *ldB)                      \
    {                                                                                                                  \
        f77_trsm<T>(NAME6, #P "trmm_", side, upLo, transA, diag, *m, *n, *alpha, A, *ldA, B, *ldB, true);              \
    }                                                                                                                  \
    void cblas_##P##trmm(enum CBLAS_ORDER order, enum CBLAS_SIDE side, enum CBLAS_UPLO upLo,                           \
                         enum CBLAS_TRANSPOSE transA, enum CBLAS_DIAG diag, int m, int n, T alpha, const T *A,         \
                         int ldA, T *B, int ldB)                                                                       \
    {                                                                                                                  \
        cblas_trsm<T>("cblas_" #P "trmm", order, side, upLo, transA, diag, m, n, alpha, A, ldA, B, ldB, true);         \
    }                                                                                                                  \
    void ulmblas_##P##trmm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE transA,                    \
                           enum CBLAS_DIAG diag, int m, int n, T alpha, const T *A, int ldA, T *B, int ldB)            \
    {                                                                                                                  \
        ulm_trsm<T>("ulmblas_" #P "trmm", side, upLo, transA, diag, m, n, alpha, A, ldA, B, ldB, true);                \
    }                                                                                                                  \
    void ATL_##P##trmm(enum CBLAS_SIDE side, enum CBLAS_UPLO upLo, enum CBLAS_TRANSPOSE transA,                        \
                       enum CBLAS_DIAG diag, int m, int n, T alpha, const T *A, int ldA, T *B, int ldB)                \
    {                                                                                                                  \
        ulmblas_##P##trmm(side, upLo, transA, diag, m, n, alpha, A, ldA, B, ldB);                                      \
    }                                                                                                                  \
    int ulmblas_gpu_##P##trmm(int right, int lower, int transA, int unit, int m, int n, T alpha, const T *dA,          \
                              int ldA, T *dB, int ldB, void *stream)                                                   \
    {                                                                                                                  \
        return trmm_device<T>(right != 0, lower != 0, transA != 0, unit != 0, m, n, alpha, dA, ldA, dB, ldB,           \
                              static_cast<hipStream_t>(stream));                                                       \
    }

ULM_TRMM_ENTRY_POINTS(d, double, "DTRMM ")
ULM_TRMM_ENTRY_POINTS(s, float, "STRMM ")

int ulmblas_gpu_dtrsm(int right, int lower, int transA, int unit, int m, int n, double alpha, const double *dA,
                      int ldA, double *dB, int ldB, void *stream)
{
    return trsm_device<double>(right != 0, lower != 0, transA != 0, unit != 0, m, n, alpha, dA, ldA, dB, ldB,
                               static_cast<hipStream_t>(stream));
}

int ulmblas_gpu_strsm(int right, int lower, int transA, int unit, int m, int n, float alpha, const float *dA,
                      int ldA, float *dB, int ldB, void *stream)
{
    return trsm_device<float>(right != 0, lower != 0, transA != 0, unit != 0, m, n, alpha, dA, ldA, dB, ldB,
                              static_cast<hipStream_t>(stream));
}

}  // extern "C"
