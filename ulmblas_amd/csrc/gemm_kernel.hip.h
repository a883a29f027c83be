// MI355X (gfx950, CDNA4) GEMM kernels: C <- alpha*op(A)*op(B) + beta*C on
// column-major operands in HBM.
//
// What each part replaces in ulmBLAS (paths relative to its source tree):
//   * gepack_A / gepack_B (ulmblas/level3/pack/gepack.tcc:40-134): the packing
//     of mc x kc / kc x nc blocks into MR / NR micro-panels becomes the staging
//     of a BM x BK tile of op(A) and a BK x BN tile of op(B) from global memory
//     into LDS, in the layout [k][m] / [k][n] whatever the transposition, with
//     zero fill past the end of k (the panels' zero padding).
//   * the NC/KC/MC frame and mgemm (ulmblas/level3/gemm.tcc:60-83,
//     ulmblas/level3/mkernel/mgemm.tcc:37-66): one workgroup per BM x BN tile of
//     C, walking k in BK slabs with two LDS stages; the whole k range is
//     accumulated in registers, so C is read and written once instead of once
//     per KC slice.
//   * ugemm (ulmblas/level3/ukernel/ref/ugemm.tcc:24-66,
//     ulmblas/level3/ukernel/sse/ugemm.tcc:60-374): the MR x NR rank-kc update
//     becomes a grid of v_mfma_f64_16x16x4_f64 / v_mfma_f32_32x32x2_f32 tiles
//     per wavefront, with the epilogue C = beta*C + alpha*AB fused and
//     beta == 0 never loading C.
//
// One kernel template, two flavours.  RAGGED = false covers a region made of
// whole BM x BN tiles and has no bounds checks at all; RAGGED = true takes any
// m x n (rows / columns past the edge are read from clamped addresses, feed
// accumulators that are never stored, and the epilogue is predicated) and
// serves the right / bottom strips and problems smaller than a tile.  Both
// share the software-pipelined main loop: global loads, LDS writes and LDS
// reads are issued in the shadow of the 64-cycle matrix instructions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace ulmgpu {

typedef double double4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// ---------------------------------------------------------------------------
// Matrix-core instruction traits.  The MFMA computes D[i][j] += sum_k
// X[i][k]*Y[k][j]; we feed X from op(B) (i runs along n) and Y from op(A)
// (j runs along m), so that consecutive lanes hold consecutive rows m of one
// column of C and the epilogue writes 128-byte runs.
//   lane l supplies X[l % W][l / W] and Y[l / W][l % W]
//   accumulator register r of lane l holds D[acc_i(r, l)][l % W]
// ---------------------------------------------------------------------------
template <typename T>
struct Mfma;

template <>
struct Mfma<double> {
    static constexpr int W = 16;   // tile edge
    static constexpr int K = 4;    // k depth of one instruction
    static constexpr int R = 4;    // accumulator values per lane
    typedef double4_t Acc;
    static __device__ __forceinline__ Acc run(double x, double y, Acc c)
    {
        return __builtin_amdgcn_mfma_f64_16x16x4f64(x, y, c, 0, 0, 0);
    }
    static __device__ __forceinline__ int acc_i(int r, int lane)
    {
        return 4 * r + (lane >> 4);
    }
};

template <>
struct Mfma<float> {
    static constexpr int W = 32;
    static constexpr int K = 2;
    static constexpr int R = 16;
    typedef float16_t Acc;
    static __device__ __forceinline__ Acc run(float x, float y, Acc c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(x, y, c, 0, 0, 0);
    }
    static __device__ __forceinline__ int acc_i(int r, int lane)
    {
        return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
    }
};

// ---------------------------------------------------------------------------
// Tile configuration.
//   BM x BN  tile of C per workgroup, BK k-slab per LDS stage
//   WM x WN  wavefronts per workgroup, each owning (BM/WM) x (BN/WN) of C
//   OCC      workgroups per CU the register budget is sized for
//   PF       k-slabs held in registers on their way from HBM to LDS (1 or 2):
//            small tiles finish a slab faster than a load from HBM returns
//            and need two in flight
//   VEC      elements per global load (1, or 16 bytes' worth: 2 doubles /
//            4 floats); the wide loads need 16-byte aligned operands and are
//            chosen by the host when base pointers and leading dimensions allow
// ---------------------------------------------------------------------------
template <typename T_, int BM_, int BN_, int BK_, int WM_, int WN_, int OCC_, int PF_ = 1, int VEC_ = 1>
struct Config {
    typedef T_ T;
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
    static constexpr int OCC = OCC_, PF = PF_, VEC = VEC_;
    static_assert(VEC == 1 || VEC * sizeof(T_) == 16, "vector loads are 16 bytes");
    static_assert(PF == 1 || PF == 2, "prefetch depth");
    static constexpr int NT = 64 * WM * WN;
    static constexpr int WAVES_PER_SIMD = (OCC * NT / 256) > 0 ? (OCC * NT / 256) : 1;
    static constexpr int W = Mfma<T>::W;
    static constexpr int WTM = BM / WM, WTN = BN / WN;   // per-wave tile
    static constexpr int TM = WTM / W, TN = WTN / W;     // MFMA tiles per wave
    // LDS row padding: consecutive k rows land 32 banks apart, so the two k
    // rows one half-wave reads (or writes) never collide.
    static constexpr int PAD = 128 / sizeof(T);
    static constexpr int LDA_S = BM + PAD, LDB_S = BN + PAD;
    static constexpr int STAGE_ELEMS = BK * (LDA_S + LDB_S);
    static constexpr size_t LDS_BYTES = 2 * STAGE_ELEMS * sizeof(T);
    // tile rows per band of the block->tile map: tall tiles take fewer rows
    static constexpr int GROUP = (BM > BN) ? 4 : 8;
    static constexpr int LA = BM * BK / NT / VEC;   // staged loads per thread
    static constexpr int LB = BN * BK / NT / VEC;
    static_assert(BM % (WM * W) == 0 && BN % (WN * W) == 0, "wave tiling");
    static_assert(BK % (2 * Mfma<T>::K) == 0, "k slab: an even number of MFMA steps");
    static_assert((BM * BK) % (NT * VEC) == 0 && (BN * BK) % (NT * VEC) == 0, "staging");
    static_assert(BM % 16 == 0 && BN % 16 == 0 && NT % 16 == 0, "staging");
};

struct GemmArgs {
    int m, n, k;
    int tiles_m, tiles_n;
    const void *A;
    const void *B;
    void *C;
    int64_t lda, ldb, ldc;
    // 0 = write the whole m x n window, +1 = only the elements on and below
    // the diagonal (row >= column), -1 = on and above.  With tri != 0:
    //  * whole-tile kernel, tri_block == 0: m == n, a multiple of BM; exactly
    //    the tiles that lie entirely inside the triangle are computed
    //    (tiles_m x tiles_n is the folded grid described in the kernel);
    //  * whole-tile kernel, tri_block > 0: the blocks of order tri_block on
    //    the diagonal of the m x m matrix (m a multiple of tri_block), stores
    //    masked element by element; the grid counts their tiles;
    //  * any-shape kernel: stores masked element by element; inside the
    //    leading tri_whole x tri_whole square it skips every tile outside the
    //    diagonal blocks of order tri_block (tri_block > 0), or every tile
    //    (tri_block < 0), or none (tri_block == 0).
    int tri;
    int tri_whole, tri_block;
    // Shared part (kernels built with SHARED = true only; sk_groups == 0: none).
    // The last sk_tiles tiles in workgroup order do not get a workgroup each:
    // their sk_tiles * ceil(k / BK) slabs are dealt evenly, as one run of
    // consecutive slabs each, to workgroups 0 .. sk_groups-1 (sk_tiles <=
    // sk_groups, so a run touches at most two tiles); the other tiles follow
    // as workgroups sk_groups, sk_groups + 1, ...  The pieces of one tile are
    // folded into C in the order of k: the first piece computes alpha*AB +
    // beta*C, every later one adds alpha*AB to what it finds, after the
    // workgroup that holds the piece before it has raised its flag.
    // A wait is bounded.  A piece whose wait runs out is not folded: its workgroup marks
    // itself beside its flag and raises no flag, so the pieces after it run out as well, and C
    // holds exactly the pieces before it.  The host follows every launch that shares tiles
    // with a second launch of the same kernel with sk_repair set: one workgroup per shared
    // tile, which looks for the first piece of its tile that gave up and, if there is one,
    // adds the product over the k range from there to the end (otherwise it ends at once).
    int sk_groups, sk_tiles;
    unsigned *sk_flags;         // one word per workgroup of the shared part, zero between launches; kSkMaxGroups words
                                // further on a second word, set to the epoch by a workgroup whose wait ran out
    unsigned sk_epoch;          // what a raised flag of this launch reads (never 0)
    unsigned sk_mute;           // testing: flags are not raised (the waits then run out)
    int sk_repair;              // this launch is the one that follows up (see above)
    long sk_spin_limit;         // polls of one wait before the workgroup gives up
    unsigned *sk_status;        // counts the waits that ran out
};

constexpr int kSkMaxGroups = 512;           // workgroups that share tiles in one launch: 256 CUs x at most 2

__device__ __forceinline__ bool in_triangle(int tri, int row, int col)
{
    return tri == 0 || (tri > 0 ? row >= col : row <= col);
}

// Workgroups are dealt to the 8 XCDs round-robin by id; give every XCD one
// contiguous run of tile numbers, and inside a run walk C in bands of GROUP
// tile rows so that the tiles resident on one XCD at a time (32 CUs) form a
// compact, roughly square block of C sharing their A and B panels through
// that XCD's 4 MiB L2.
template <int GROUP>
__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n,
                                              int &tm, int &tn)
{
    constexpr int XCDS = 8;
    const int total = tiles_m * tiles_n;
    int id = bid;
    if (total >= 2 * XCDS) {
        const int per = (total + XCDS - 1) / XCDS;
        const int tall = (total % XCDS == 0) ? XCDS : total % XCDS;
        const int xcd = bid % XCDS, slot = bid / XCDS;
        id = (xcd < tall) ? xcd * per + slot
                          : tall * per + (xcd - tall) * (per - 1) + slot;
    }
    const int in_group = GROUP * tiles_n;
    const int g = id / in_group;
    const int first = g * GROUP;
    const int gsize = min(tiles_m - first, GROUP);
    const int r = id - g * in_group;
    tm = first + r % gsize;
    tn = r / gsize;
}

// ---------------------------------------------------------------------------
// Staging pattern: an X x BK tile of op(A) or op(B) over NT threads, VEC
// elements (contiguous in memory) per load.  Load i of thread t starts at
// (x0(t) + dx(i), k0(t) + dk(i)) with compile-time dx, dk, so its global
// address is a per-thread offset plus a uniform one and its LDS address a
// per-thread base plus an immediate.
//   contiguous along x in memory (A as stored, B transposed): a wavefront
//     reads 64*VEC consecutive x of one k row and writes them to LDS as they
//     are;
//   contiguous along k in memory (A transposed, B as stored): a wavefront
//     reads 16 x-lines, 4*VEC consecutive k of each, and its LDS writes go to
//     16 consecutive x per k row (the transposition happens here).
// ---------------------------------------------------------------------------
template <int X, int BK, int NT, bool KCONTIG, int VEC>
struct Stage {
    static constexpr int L = X * BK / NT / VEC;
    static constexpr int XV = X / VEC;                   // x-contiguous: vectors per k row
    static constexpr bool XC_SMALL = (NT % XV == 0);     //   several k rows per pass
    static constexpr int KV = BK / VEC;                  // k-contiguous: vectors per x line
    static constexpr int KROWS = NT / 16;                //   k vectors covered per pass
    static constexpr bool KC_SMALL = (KROWS % KV == 0);  //   a pass covers the whole k range
    static_assert(X % VEC == 0 && BK % VEC == 0, "staging pattern");
    static_assert(KCONTIG ? (KC_SMALL || KV % KROWS == 0) : (XC_SMALL || XV % NT == 0), "staging pattern");
    static __device__ __forceinline__ int x0(int t)
    {
        if (!KCONTIG) return VEC * (XC_SMALL ? t % XV : t);
        return KC_SMALL ? (t % 16) + 16 * ((t / 16) / KV) : (t % 16);
    }
    static __device__ __forceinline__ int k0(int t)
    {
        if (!KCONTIG) return XC_SMALL ? t / XV : 0;
        return VEC * (KC_SMALL ? (t / 16) % KV : (t / 16));
    }
    static constexpr int dx(int i)
    {
        if (!KCONTIG) return XC_SMALL ? 0 : VEC * NT * (i % (XV / NT));
        return KC_SMALL ? 16 * (KROWS / KV) * i : 16 * (i / (KV / KROWS));
    }
    static constexpr int dk(int i)
    {
        if (!KCONTIG) return XC_SMALL ? (NT / XV) * i : i / (XV / NT);
        return KC_SMALL ? 0 : VEC * KROWS * (i % (KV / KROWS));
    }
    // true when every load of a thread has the same x (then one clamp serves all)
    static constexpr bool SAME_X = !KCONTIG && XC_SMALL;
};

// VEC consecutive elements as one register value
template <typename T, int VEC>
struct Packet {
    typedef T type __attribute__((ext_vector_type(VEC)));
    static __device__ __forceinline__ T get(const type &v, int e) { return v[e]; }
    static __device__ __forceinline__ void set(type &v, int e, T x) { v[e] = x; }
    static __device__ __forceinline__ type zero()
    {
        type v;
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[e] = T(0);
        return v;
    }
};
template <typename T>
struct Packet<T, 1> {
    typedef T type;
    static __device__ __forceinline__ T get(const type &v, int) { return v; }
    static __device__ __forceinline__ void set(type &v, int, T x) { v = x; }
    static __device__ __forceinline__ type zero() { return T(0); }
};

// A stretch of global memory as a buffer: the origin (uniform over the
// workgroup) sits in four scalar registers, a load names a 32-bit byte offset
// from it (at most 4 GiB - 1; no bounds are checked: the range is left open).
// VT: what one load fetches (4, 8 or 16 bytes).
template <typename VT>
struct BufferOf {
    __amdgpu_buffer_rsrc_t rsrc;
    __device__ __forceinline__ explicit BufferOf(const void *origin)
    {
        // (0x00020000: dword 3 of a raw buffer descriptor on gfx9 - 32-bit data format, no swizzle)
        rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(origin), 0, -1, 0x00020000);
    }
    __device__ __forceinline__ VT load(uint32_t offset) const
    {
        if constexpr (sizeof(VT) == 16) {
            typedef int v4 __attribute__((ext_vector_type(4)));
            return __builtin_bit_cast(VT, (v4)__builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)offset, 0, 0));
        } else if constexpr (sizeof(VT) == 8) {
            typedef int v2 __attribute__((ext_vector_type(2)));
            return __builtin_bit_cast(VT, (v2)__builtin_amdgcn_raw_buffer_load_b64(rsrc, (int)offset, 0, 0));
        } else {
            return __builtin_bit_cast(VT, (int)__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)offset, 0, 0));
        }
    }
};

// Scheduling recipe for one group of NMFMA matrix instructions: after each
// MFMA let the wave issue up to one LDS read (NDSR in total) and an even share
// of NDSW LDS writes and NVMEM global loads, so that these run while the
// matrix pipe (64 cycles per instruction) is busy.
template <int NMFMA, int NDSR, int NDSW, int NVMEM>
__device__ __forceinline__ void interleave_with_mfma()
{
    constexpr int DSW_PER = (NDSW + NMFMA - 1) / NMFMA;
    constexpr int VMEM_PER = (NVMEM + NMFMA - 1) / NMFMA;
#pragma unroll
    for (int q = 0; q < NMFMA; ++q) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                  // 1 MFMA
        if (q < NDSR) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);    // 1 DS read
        if (NDSW > 0) __builtin_amdgcn_sched_group_barrier(0x200, DSW_PER, 0);
        if (NVMEM > 0) __builtin_amdgcn_sched_group_barrier(0x020, VMEM_PER, 0);
    }
}

// Workgroup `tile` of the launch that follows up on a launch with shared tiles
// looks after shared tile `tile`.  The pieces of that tile that had to wait
// are those of the workgroups b whose run of slabs begins inside the tile; the
// first of them that gave up (all after it did so too) says from which slab on
// the tile's product is still missing (-1: from none).  `word`: a place in LDS.
__device__ __forceinline__ int first_slab_missing(const GemmArgs &args, int tile, int slabs_of_tile, int *word)
{
    if (threadIdx.x == 0) {
        const long G = args.sk_groups;
        const long units = (long)args.sk_tiles * slabs_of_tile;
        const long lo = (long)tile * slabs_of_tile, hi = lo + slabs_of_tile;
        int from = -1;
        for (long b = lo * G / units; b < G; ++b) {
            const long u = units * b / G;
            if (u <= lo) continue;
            if (u >= hi) break;
            if (from < 0 && __hip_atomic_load(args.sk_flags + kSkMaxGroups + b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == args.sk_epoch)
                from = (int)(u - lo);
            if (from >= 0) {    // as the next launch expects them (a flag may have been raised late)
                __hip_atomic_store(args.sk_flags + kSkMaxGroups + b, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(args.sk_flags + (b - 1), 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        *word = from;
    }
    __syncthreads();
    const int from = *word;
    __syncthreads();            // the word's place belongs to the first slab from here on
    return from;
}

// The kernel.  Preconditions (checked by the host): k >= 1, m, n >= 1, and for
// RAGGED = false m % BM == 0, n % BN == 0.  Per slab of BK: S = BK / MFMA_K
// steps of TM*TN MFMAs; the fragments of step s+1 are read from LDS while
// step s runs (register double buffer), the next PF slabs but one are in
// flight from global memory, the slab one ahead is written to the other LDS
// stage during step S-2, and one barrier per slab separates that write from
// the first read of the stage.
// FOLLOWUP (SHARED kernels only): the instantiation for the launch that follows a launch with
// shared tiles (GemmArgs::sk_repair); the launch itself uses the other one, which is not slowed
// by code it never runs.
template <class CFG, bool TRANSA, bool TRANSB, bool RAGGED, bool SHARED = false, bool FOLLOWUP = false>
__global__ void
__attribute__((amdgpu_flat_work_group_size(CFG::NT, CFG::NT),
               amdgpu_waves_per_eu(CFG::WAVES_PER_SIMD, CFG::WAVES_PER_SIMD)))
gemm_kernel(GemmArgs args, typename CFG::T alpha, typename CFG::T beta_arg)
{
    typedef typename CFG::T T;
    typedef Mfma<T> MF;
    typedef typename MF::Acc Acc;
    constexpr int BM = CFG::BM, BN = CFG::BN, BK = CFG::BK, NT = CFG::NT;
    constexpr int W = MF::W, TM = CFG::TM, TN = CFG::TN;
    constexpr int LA = CFG::LA, LB = CFG::LB;
    constexpr int S = BK / MF::K;
    // op(A)[m][k]: as stored, m is contiguous; transposed, k is contiguous.
    // op(B)[k][n]: as stored, k is contiguous; transposed, n is contiguous.
    constexpr bool A_KCONTIG = TRANSA, B_KCONTIG = !TRANSB;
    constexpr int VEC = CFG::VEC;
    static_assert(!RAGGED || VEC == 1, "the any-shape kernel loads element by element");
    static_assert(!(RAGGED && SHARED), "tiles are shared between workgroups by the whole-tile kernel only");
    static_assert(SHARED || !FOLLOWUP, "only launches with shared tiles are followed up");
    // How the kernels that take tiles past the edge of C fetch whole slabs.  The two largest tiles (256 x 128
    // fp64, 256 x 256 fp32: eight wavefronts, a slab of 8192 matrix-pipe cycles) through global loads at
    // 64-bit addresses, every packet along x passed through the selects that put an edge tile's packets in
    // place (the compiler places those, and the wait for the loads, at the top of the iteration, which these
    // tiles do not feel).  The smaller ones, whose slabs are too short for that: buffer loads (a descriptor
    // in scalar registers plus a 32-bit offset per packet), and the k loop twice, so that tiles inside C
    // skip the selects and tiles past the edge keep them next to the LDS writes.  Measured, one launch over
    // all of C against whole tiles of the same count, A as stored: 128 x 128 fp64 1.17 -> 1.06, both
    // operands along k 1.04 -> 1.00; the two largest tiles lose 5 % that way and stay as they were.
    constexpr bool BUFFERED = SHARED && (size_t)BM * BN * sizeof(T) <= 131072;
    // The whole-tile kernels with 16-byte loads fetch the same way, up to the same tile size (the host sees to
    // it that a slab of a tile spans less than 4 GiB): no 64-bit address is worked out per load and none is
    // held in registers across the loop.
    // (not the 128 x 128 fp64 tile: alone on its CU it gains 2 % by it - 2048^3 -, with a second workgroup
    // beside it, as in every launch of several rounds, it loses 4 - 8 %: 6144 x 6016 x 2048 2.11 -> 2.28 ms)
    constexpr bool PLAINBUF = !SHARED && !RAGGED && VEC > 1 && (size_t)BM * BN * sizeof(T) <= 131072 &&
                              !(sizeof(T) == 8 && BM == 128 && BN == 128);
    typedef Stage<BM, BK, NT, A_KCONTIG, VEC> SA;
    typedef Stage<BN, BK, NT, B_KCONTIG, VEC> SB;
    typedef Packet<T, VEC> PK;
    typedef typename PK::type VT;
    // the same packet at the alignment of one element: a 16-byte load the hardware carries out at any
    // element-aligned address
    typedef VT VTU __attribute__((aligned(sizeof(T))));

    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    T *lds = reinterpret_cast<T *>(lds_raw);

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = t >> 6;
    const int wm = wave % CFG::WM, wn = wave / CFG::WM;

    // The pieces of work of this workgroup: a tile (by its number in workgroup
    // order) and a range of its k slabs.  Without sharing: one piece, the
    // whole tile.
    int pt0 = (int)blockIdx.x, pt1 = 0, pb0 = 0, pb1 = 0, pe0 = 0, pe1 = 0;     // tile, first slab, end slab of pieces 0 and 1
    int npieces = 1;
    const int slabs_of_tile = (args.k + BK - 1) / BK;
    pe0 = slabs_of_tile;
    if constexpr (SHARED) {
        const int G = args.sk_groups, bid = (int)blockIdx.x;
        if (G > 0) {
            const int first_shared = args.tiles_m * args.tiles_n - args.sk_tiles;
            if constexpr (FOLLOWUP) {
                const int from = first_slab_missing(args, bid, slabs_of_tile, reinterpret_cast<int *>(lds_raw));
                if (from < 0) return;
                pt0 = first_shared + bid;
                pb0 = from;
            } else if (bid >= G) {
                pt0 = bid - G;
            } else {
                const long units = (long)args.sk_tiles * slabs_of_tile;
                const long u0 = units * bid / G, u1 = units * (bid + 1) / G;     // u1 > u0: the host sees to it
                const int t0 = (int)(u0 / slabs_of_tile), t1 = (int)((u1 - 1) / slabs_of_tile);
                if (t0 == t1) {
                    pt0 = first_shared + t0;
                    pb0 = (int)(u0 - (long)t0 * slabs_of_tile);
                    pe0 = (int)(u1 - (long)t0 * slabs_of_tile);
                } else {
                    // the head of the later tile first: the workgroup that finishes that tile waits for it
                    npieces = 2;
                    pt0 = first_shared + t1;
                    pb0 = 0;
                    pe0 = (int)(u1 - (long)t1 * slabs_of_tile);
                    pt1 = first_shared + t0;
                    pb1 = (int)(u0 - (long)t0 * slabs_of_tile);
                    pe1 = slabs_of_tile;
                }
            }
        }
    }
    for (int piece = 0; piece < npieces; ++piece) {
    // the stages of LDS are about to be written again: every wavefront must be done reading them
    if (SHARED && piece > 0) __syncthreads();
    const int slab_begin = piece == 0 ? pb0 : pb1, slab_end = piece == 0 ? pe0 : pe1;
    const T beta = (SHARED && slab_begin > 0) ? T(1) : beta_arg;
    int tile_m, tile_n;
    tile_of_block<CFG::GROUP>(piece == 0 ? pt0 : pt1, args.tiles_m, args.tiles_n, tile_m, tile_n);
    if (args.tri != 0) {
        if constexpr (RAGGED) {
            // a tile that lies entirely in the triangle that is not written has nothing to do
            const int m0 = tile_m * BM, n0 = tile_n * BN;
            if (args.tri > 0 && m0 + BM - 1 < n0) return;
            if (args.tri < 0 && m0 > n0 + BN - 1) return;
            if (args.tri_block > 0 && m0 < args.tri_whole && n0 < args.tri_whole &&
                m0 / args.tri_block != n0 / args.tri_block) return;
            if (args.tri_block < 0 && m0 < args.tri_whole && n0 < args.tri_whole) return;
        } else if (args.tri_block > 0) {
            // The blocks of order tri_block on the diagonal, tile by tile: workgroup ids count
            // the tiles of block 0, then of block 1, ...; tiles in the other triangle exit,
            // the rest mask their stores element by element.
            const int tpm = args.tri_block / BM, tpn = args.tri_block / BN;
            const int blk = blockIdx.x / (tpm * tpn), r = blockIdx.x % (tpm * tpn);
            tile_m = blk * tpm + r % tpm;
            tile_n = blk * tpn + r / tpm;
            if (args.tri > 0 ? (tile_m * BM + BM - 1 < tile_n * BN) : (tile_n * BN + BN - 1 < tile_m * BM)) return;
        } else {
            // The grid holds only the tiles that lie entirely inside the
            // triangle of the T x cT tile grid (T = m / BM tile rows, c = BM /
            // BN): row i of the lower triangle has its first c*i tiles there,
            // so rows p and T-1-p together make one row of W = c*(T-1) tiles
            // and the launch is a rectangle of ceil(T/2) such rows (tiles_m)
            // by W (tiles_n).  The upper triangle is the point reflection.
            // (launched only for variants whose BM is a multiple of BN)
            constexpr int c = BM >= BN ? BM / BN : 1;
            const int T = args.m / BM;
            const int p = tile_m, q = tile_n;
            int i = p, j = q;
            if (q >= c * p) {
                i = T - 1 - p;
                j = q - c * p;
                if (i == p) return;      // odd T: the middle row has no partner (the host lets workgroups
                                         // share tiles of such a launch only when T is even)
            }
            if (args.tri < 0) {
                i = T - 1 - i;
                j = c * T - 1 - j;
            }
            tile_m = i;
            tile_n = j;
        }
    }
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int M = args.m, N = args.n;
    // this piece's share of k, counted from its first slab
    const int K = SHARED ? min(args.k, slab_end * BK) - slab_begin * BK : args.k;

    const int64_t a_sx = TRANSA ? args.lda : 1, a_sk = TRANSA ? 1 : args.lda;
    const int64_t b_sx = TRANSB ? 1 : args.ldb, b_sk = TRANSB ? args.ldb : 1;
    // uniform pointers to the tile's first slab
    const T *a_base = static_cast<const T *>(args.A) + (int64_t)m0 * a_sx + (SHARED ? (int64_t)slab_begin * BK * a_sk : 0);
    const T *b_base = static_cast<const T *>(args.B) + (int64_t)n0 * b_sx + (SHARED ? (int64_t)slab_begin * BK * b_sk : 0);

    // Per-thread element offsets of the staged loads inside a slab.  Whole
    // tiles: one offset per operand plus compile-time multiples of the
    // strides.  Ragged tiles: the x coordinate of every load is clamped to the
    // last valid row / column, so nothing outside the operand is touched; the
    // duplicated data only reaches accumulators that are never stored.
    // SHARED kernels take any m x n as well: a tile that reaches past the edge of C (uniform per
    // tile) masks its stores.
    const bool edge = SHARED && (m0 + BM > M || n0 + BN > N);
    const int xa_last = min(BM, M - m0) - 1, xb_last = min(BN, N - n0) - 1;     // last valid row / column of the tile
    constexpr int NOA = (RAGGED && !SA::SAME_X) ? LA : 1;
    constexpr int NOB = (RAGGED && !SB::SAME_X) ? LB : 1;
    int64_t a_voff[NOA], b_voff[NOB];
    // SHARED kernels: the byte offset of every packet from the slab's (uniform) origin, 32 bits
    // each (the host sees to it that a tile's slab spans less than 4 GiB), worked out once per
    // tile.  They also take tiles that reach past the edge of C, without a branch in the k
    // loop: an operand read in packets along k reads, for a line past the edge, the last valid
    // line; an operand read in packets along x has all packets of a thread at the same x, and
    // that x is moved back until the packet ends on the last valid element (the host sees to it
    // that this does not leave the tile), and what a packet read is moved up again by as many
    // places (a_shift, b_shift), so that every valid element sits where the unclamped packet
    // would have put it.  Places past the edge hold values that only reach accumulators nobody
    // stores.
    constexpr int NSA = (SHARED || PLAINBUF) ? LA : 1, NSB = (SHARED || PLAINBUF) ? LB : 1;
    // A packet along x that is moved back may begin up to VEC-1 places before the tile (in the
    // tile row or column before it; the host sees to it that there is one, or that the first
    // tile holds a whole packet): offsets are unsigned, so they count from that far back.
    constexpr int A_XBIAS = A_KCONTIG ? 0 : VEC - 1, B_XBIAS = B_KCONTIG ? 0 : VEC - 1;
    uint32_t a_off32[NSA], b_off32[NSB];
    int a_shift = 0, b_shift = 0;
    if constexpr (SHARED) {
        static_assert(!SHARED || ((A_KCONTIG || SA::SAME_X) && (B_KCONTIG || SB::SAME_X)),
                      "packets along x: one x per thread");
#pragma unroll
        for (int i = 0; i < LA; ++i) {
            const int x = A_KCONTIG ? min(SA::x0(t) + SA::dx(i), xa_last) : min(SA::x0(t), xa_last + 1 - VEC);
            if (!A_KCONTIG) a_shift = SA::x0(t) - x;
            // x >= 1 - VEC: the offsets count from VEC-1 places before the tile's origin (XBIAS)
            a_off32[i] = (uint32_t)(((int64_t)(x + A_XBIAS) * a_sx + (int64_t)(SA::k0(t) + SA::dk(i)) * a_sk) * (int64_t)sizeof(T));
        }
#pragma unroll
        for (int i = 0; i < LB; ++i) {
            const int x = B_KCONTIG ? min(SB::x0(t) + SB::dx(i), xb_last) : min(SB::x0(t), xb_last + 1 - VEC);
            if (!B_KCONTIG) b_shift = SB::x0(t) - x;
            b_off32[i] = (uint32_t)(((int64_t)(x + B_XBIAS) * b_sx + (int64_t)(SB::k0(t) + SB::dk(i)) * b_sk) * (int64_t)sizeof(T));
        }
        a_voff[0] = b_voff[0] = 0;
    } else if constexpr (PLAINBUF) {
#pragma unroll
        for (int i = 0; i < LA; ++i)
            a_off32[i] = (uint32_t)(((int64_t)(SA::x0(t) + SA::dx(i)) * a_sx + (int64_t)(SA::k0(t) + SA::dk(i)) * a_sk) * (int64_t)sizeof(T));
#pragma unroll
        for (int i = 0; i < LB; ++i)
            b_off32[i] = (uint32_t)(((int64_t)(SB::x0(t) + SB::dx(i)) * b_sx + (int64_t)(SB::k0(t) + SB::dk(i)) * b_sk) * (int64_t)sizeof(T));
        a_voff[0] = (int64_t)SA::x0(t) * a_sx + (int64_t)SA::k0(t) * a_sk;       // (the last, partial slab still goes by address)
        b_voff[0] = (int64_t)SB::x0(t) * b_sx + (int64_t)SB::k0(t) * b_sk;
    } else {
        const int xa_max = RAGGED ? min(BM, M - m0) - 1 : BM - 1;
        const int xb_max = RAGGED ? min(BN, N - n0) - 1 : BN - 1;
#pragma unroll
        for (int i = 0; i < NOA; ++i) {
            const int x = RAGGED ? min(SA::x0(t) + (NOA > 1 ? SA::dx(i) : 0), xa_max) : SA::x0(t);
            a_voff[i] = (int64_t)x * a_sx + (int64_t)(SA::k0(t) + (NOA > 1 ? SA::dk(i) : 0)) * a_sk;
        }
#pragma unroll
        for (int i = 0; i < NOB; ++i) {
            const int x = RAGGED ? min(SB::x0(t) + (NOB > 1 ? SB::dx(i) : 0), xb_max) : SB::x0(t);
            b_voff[i] = (int64_t)x * b_sx + (int64_t)(SB::k0(t) + (NOB > 1 ? SB::dk(i) : 0)) * b_sk;
        }
    }
    auto a_elem = [&](const T *slab, int i) -> const T * {
        if (NOA > 1) return slab + a_voff[i];
        return slab + a_voff[0] + (int64_t)SA::dx(i) * a_sx + (int64_t)SA::dk(i) * a_sk;
    };
    auto b_elem = [&](const T *slab, int i) -> const T * {
        if (NOB > 1) return slab + b_voff[i];
        return slab + b_voff[0] + (int64_t)SB::dx(i) * b_sx + (int64_t)SB::dk(i) * b_sk;
    };

    constexpr int PF = CFG::PF;
    VT ra[PF][LA], rb[PF][LB];

    // what a packet read along x, moved up by `shift` places (see a_shift above)
    auto moved_up = [&](VT v, int shift) -> VT {
        if constexpr (VEC == 1) {
            return v;
        } else {
            VT out;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                T val = PK::get(v, VEC - 1);
#pragma unroll
                for (int j = VEC - 2; j >= e; --j) val = (e + shift == j) ? PK::get(v, j) : val;
                PK::set(out, e, val);
            }
            return out;
        }
    };
    auto load_whole = [&](auto set_c, int slab) {
        constexpr int SET = decltype(set_c)::value;
        const T *ab = a_base + (int64_t)slab * BK * a_sk;
        const T *bb = b_base + (int64_t)slab * BK * b_sk;
        if constexpr (SHARED) {
            if constexpr (BUFFERED) {
                // buffer loads: the slab's origin (uniform) travels in scalar registers as a buffer
                // descriptor, the packet's place as a 32-bit offset, so no 64-bit address is made per load
                const BufferOf<VT> abuf(ab - A_XBIAS * a_sx), bbuf(bb - B_XBIAS * b_sx);
#pragma unroll
                for (int i = 0; i < LA; ++i) ra[SET][i] = abuf.load(a_off32[i]);
#pragma unroll
                for (int i = 0; i < LB; ++i) rb[SET][i] = bbuf.load(b_off32[i]);
            } else {
                const char *ac = reinterpret_cast<const char *>(ab - A_XBIAS * a_sx);
                const char *bc = reinterpret_cast<const char *>(bb - B_XBIAS * b_sx);
#pragma unroll
                for (int i = 0; i < LA; ++i) ra[SET][i] = *reinterpret_cast<const VTU *>(ac + a_off32[i]);
#pragma unroll
                for (int i = 0; i < LB; ++i) rb[SET][i] = *reinterpret_cast<const VTU *>(bc + b_off32[i]);
            }
            return;
        }
        if constexpr (PLAINBUF) {
            const BufferOf<VT> abuf(ab), bbuf(bb);
#pragma unroll
            for (int i = 0; i < LA; ++i) ra[SET][i] = abuf.load(a_off32[i]);
#pragma unroll
            for (int i = 0; i < LB; ++i) rb[SET][i] = bbuf.load(b_off32[i]);
            return;
        }
#pragma unroll
        for (int i = 0; i < LA; ++i) ra[SET][i] = *reinterpret_cast<const VTU *>(a_elem(ab, i));
#pragma unroll
        for (int i = 0; i < LB; ++i) rb[SET][i] = *reinterpret_cast<const VTU *>(b_elem(bb, i));
    };
    // the last, partial slab: k rows past K count as zero (the zero padding of
    // the reference's packed panels, ulmblas/level3/pack/gepack.tcc:59-70);
    // read element by element, so that nothing past the end of k is touched
    auto load_tail = [&](auto set_c, int slab) {
        constexpr int SET = decltype(set_c)::value;
        const int kbase = slab * BK;
        const T *ab = a_base + (int64_t)slab * BK * a_sk;
        const T *bb = b_base + (int64_t)slab * BK * b_sk;
#pragma unroll
        for (int i = 0; i < LA; ++i) {
            const T *p = a_elem(ab, i);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const int kk = SA::k0(t) + SA::dk(i) + (A_KCONTIG ? e : 0);
                const bool ok = kbase + kk < K;
                if constexpr (SHARED) {     // the elements of the packet of a whole slab, one by one
                    const T *q = reinterpret_cast<const T *>(reinterpret_cast<const char *>(ab - A_XBIAS * a_sx) + a_off32[i]);
                    PK::set(ra[SET][i], e, ok ? q[e] : T(0));
                } else {
                    PK::set(ra[SET][i], e, ok ? p[e] : T(0));
                }
            }
        }
#pragma unroll
        for (int i = 0; i < LB; ++i) {
            const T *p = b_elem(bb, i);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const int kk = SB::k0(t) + SB::dk(i) + (B_KCONTIG ? e : 0);
                const bool ok = kbase + kk < K;
                if constexpr (SHARED) {
                    const T *q = reinterpret_cast<const T *>(reinterpret_cast<const char *>(bb - B_XBIAS * b_sx) + b_off32[i]);
                    PK::set(rb[SET][i], e, ok ? q[e] : T(0));
                } else {
                    PK::set(rb[SET][i], e, ok ? p[e] : T(0));
                }
            }
        }
    };

    // registers -> LDS stage, layout As[kk][m], Bs[kk][n]: a packet read along
    // x is stored as it is, a packet read along k goes to VEC consecutive rows
    const int a_soff = SA::k0(t) * CFG::LDA_S + SA::x0(t);
    const int b_soff = SB::k0(t) * CFG::LDB_S + SB::x0(t);
    auto store_slab = [&](auto set_c, int stage, auto edge_c) {
        constexpr int SET = decltype(set_c)::value;
        constexpr bool MOVE = SHARED && decltype(edge_c)::value;     // packets along x of a tile past the edge
        // (the selects that move such packets must not travel up the iteration: the wait for the global
        // loads whose data they take would travel with them; everything else may pass this point)
        if constexpr (BUFFERED && MOVE && VEC > 1 && (!A_KCONTIG || !B_KCONTIG)) __builtin_amdgcn_sched_barrier(0x7fc);
        T *As = lds + stage * CFG::STAGE_ELEMS + a_soff;
        T *Bs = lds + stage * CFG::STAGE_ELEMS + BK * CFG::LDA_S + b_soff;
#pragma unroll
        for (int i = 0; i < LA; ++i) {
            T *q = As + SA::dk(i) * CFG::LDA_S + SA::dx(i);
            if (!A_KCONTIG) {
                // (the move is made here, where the packet is needed, not where it was asked for)
                *reinterpret_cast<VT *>(q) = MOVE ? moved_up(ra[SET][i], a_shift) : ra[SET][i];
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e) q[e * CFG::LDA_S] = PK::get(ra[SET][i], e);
            }
        }
#pragma unroll
        for (int i = 0; i < LB; ++i) {
            T *q = Bs + SB::dk(i) * CFG::LDB_S + SB::dx(i);
            if (!B_KCONTIG) {
                *reinterpret_cast<VT *>(q) = MOVE ? moved_up(rb[SET][i], b_shift) : rb[SET][i];
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e) q[e * CFG::LDB_S] = PK::get(rb[SET][i], e);
            }
        }
    };

    Acc acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < MF::R; ++r) acc[i][j][r] = T(0);

    // this lane's fragment origin inside a stage
    const int frag_k = lane / W, frag_x = lane % W;
    const int a_off = frag_k * CFG::LDA_S + wm * CFG::WTM + frag_x;
    const int b_off = frag_k * CFG::LDB_S + wn * CFG::WTN + frag_x;

    T fa[2][TM], fb[2][TN];
    auto read_frags = [&](int buf, int stage, int s) {
        const T *As = lds + stage * CFG::STAGE_ELEMS + a_off + s * MF::K * CFG::LDA_S;
        const T *Bs = lds + stage * CFG::STAGE_ELEMS + BK * CFG::LDA_S + b_off + s * MF::K * CFG::LDB_S;
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[buf][i] = As[i * W];
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[buf][j] = Bs[j * W];
    };
    auto mfma_group = [&](int buf) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int i = 0; i < TM; ++i) acc[i][j] = MF::run(fb[buf][j], fa[buf][i], acc[i][j]);
    };

    // LDS write instructions per slab (a packet read along k takes VEC of them)
    constexpr int NDSW = LA * (A_KCONTIG ? VEC : 1) + LB * (B_KCONTIG ? VEC : 1);
    const int nwhole = K / BK;
    const int nslabs = (K + BK - 1) / BK;
    auto load_any = [&](auto set_c, int slab) {
        if (slab < nwhole) load_whole(set_c, slab); else load_tail(set_c, slab);
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;

    // The k loop exists twice in the kernels that take tiles past the edge of C: tiles that lie inside C
    // (all but the last row and column of tiles) do not pay for moving packets on their way into LDS -
    // a few selects per slab, but the compiler places them, and with them the wait for the global loads
    // they consume, at the top of the iteration.
    auto k_loop = [&](auto edge_c) {
        // Slab j travels through register set j % PF and LDS stage j % 2.  One
        // iteration multiplies slab kb out of LDS stage STAGE = kb % 2 and, around
        // its last two MFMA steps, moves slab kb+1 from registers to the other
        // stage and starts the load of slab kb+1+PF into the registers just freed.
        // STEADY: both of those slabs exist and the loaded one is whole.
        auto iteration = [&](auto stage_c, auto set_c, auto steady_c, int kb) {
            constexpr int STAGE = decltype(stage_c)::value;
            constexpr bool STEADY = decltype(steady_c)::value != 0;
            typedef decltype(set_c) Set;                // register set (kb + 1) % PF
    #pragma unroll
            for (int s = 0; s + 2 < S; ++s) {
                read_frags((s + 1) & 1, STAGE, s + 1);
                mfma_group(s & 1);
                if (STEADY) interleave_with_mfma<TM * TN, TM + TN, 0, 0>();
            }
            read_frags((S - 1) & 1, STAGE, S - 1);
            mfma_group((S - 2) & 1);
            if (STEADY || kb + 1 < nslabs) store_slab(Set(), STAGE ^ 1, edge_c);
            if (STEADY) interleave_with_mfma<TM * TN, TM + TN, NDSW, 0>();
            __syncthreads();
            if (STEADY) load_whole(Set(), kb + 1 + PF);
            else if (kb + 1 + PF < nslabs) load_any(Set(), kb + 1 + PF);
            if (STEADY || kb + 1 < nslabs) read_frags(0, STAGE ^ 1, 0);
            mfma_group((S - 1) & 1);
            if (STEADY) interleave_with_mfma<TM * TN, TM + TN, 0, LA + LB>();
        };

        load_any(I0(), 0);
        store_slab(I0(), 0, edge_c);
        if constexpr (PF == 2) {
            if (1 < nslabs) load_any(I1(), 1);
            if (2 < nslabs) load_any(I0(), 2);
            __syncthreads();
            read_frags(0, 0, 0);
            int kb = 0;
            for (; kb + 2 + PF < nwhole; kb += 2) {
                iteration(I0(), I1(), I1(), kb);
                iteration(I1(), I0(), I1(), kb + 1);
            }
            for (; kb < nslabs; ++kb) {
                if (kb & 1) iteration(I1(), I0(), I0(), kb);
                else iteration(I0(), I1(), I0(), kb);
            }
        } else {
            // one register set: the LDS stage is a run-time value and the loop is
            // not unrolled over stages, which keeps the accumulators of the large
            // tiles in place (unrolling makes the compiler spill them)
            if (1 < nslabs) load_any(I0(), 1);
            __syncthreads();
            read_frags(0, 0, 0);
            int kb = 0;
            for (; kb + 2 < nwhole; ++kb) {
                const int cur = kb & 1;
    #pragma unroll
                for (int s = 0; s + 2 < S; ++s) {
                    read_frags((s + 1) & 1, cur, s + 1);
                    mfma_group(s & 1);
                    interleave_with_mfma<TM * TN, TM + TN, 0, 0>();
                }
                read_frags((S - 1) & 1, cur, S - 1);
                mfma_group((S - 2) & 1);
                store_slab(I0(), cur ^ 1, edge_c);
                interleave_with_mfma<TM * TN, TM + TN, NDSW, 0>();
                __syncthreads();
                load_whole(I0(), kb + 2);
                read_frags(0, cur ^ 1, 0);
                mfma_group((S - 1) & 1);
                interleave_with_mfma<TM * TN, TM + TN, 0, LA + LB>();
            }
            for (; kb < nslabs; ++kb) {
                const int cur = kb & 1;
    #pragma unroll
                for (int s = 0; s + 1 < S; ++s) {
                    read_frags((s + 1) & 1, cur, s + 1);
                    mfma_group(s & 1);
                }
                if (kb + 1 < nslabs) store_slab(I0(), cur ^ 1, edge_c);
                __syncthreads();
                if (kb + 2 < nslabs) load_any(I0(), kb + 2);
                if (kb + 1 < nslabs) read_frags(0, cur ^ 1, 0);
                mfma_group((S - 1) & 1);
            }
        }
    };
    if constexpr (BUFFERED) {
        if (edge) k_loop(std::true_type{}); else k_loop(std::false_type{});
    } else {
        k_loop(std::true_type{});
    }

    // epilogue: C = beta*C + alpha*AB on the m x n window only; beta == 0
    // stores without loading (ulmblas/level3/ukernel/ref/ugemm.tcc:40-45); C is
    // fetched in batches of rows, one batch ahead of the one being combined.
    T *__restrict__ Cg = static_cast<T *>(args.C);
    const int mrow = m0 + wm * CFG::WTM + frag_x;
    const int ncol = n0 + wn * CFG::WTN;
    constexpr int RB = MF::R < 4 ? MF::R : 4;     // accumulator rows per batch
    constexpr int NBATCH = TN * (MF::R / RB);
    // batch b covers column group j = b / (R/RB), accumulator rows r0 .. r0+RB-1
    // `masked`: whether stores (and fetches) are predicated element by element.
    // The any-shape kernel always is; the whole-tile kernel only for the
    // triangular launches, in a copy of this code that plain products never enter.
    // `through`: C is read and written past the caches that the GPU's dies do
    // not share (loads and stores of device scope), because another workgroup,
    // possibly on another die, wrote these elements a moment ago or will read
    // them in a moment; only pieces of shared tiles come here.
    // (the lane number the epilogue works with is tied to the piece by a term that is always
    // zero: otherwise the column offsets of all accumulators, which depend on the lane alone,
    // are worked out once before the loop over the pieces and held in registers across the k
    // loop, where the accumulators need every register)
    const int elane = SHARED ? (lane | (slab_begin >> 30)) : lane;
    auto fused = [](T a, T b, T c) -> T {
        if constexpr (sizeof(T) == 8) return __builtin_fma(a, b, c);
        else return __builtin_fmaf(a, b, c);
    };
    auto epilogue = [&](auto masked_c, auto through_c) {
        constexpr bool MASKED = decltype(masked_c)::value;
        constexpr bool THROUGH = decltype(through_c)::value;
        T cbuf[2][RB][TM];
        auto keep = [&](int row, int nn) {
            if constexpr (!MASKED) return true;
            else if constexpr (RAGGED) return nn < N && row < M && in_triangle(args.tri, row, nn);
            else if constexpr (SHARED) return nn < N && row < M;
            else return in_triangle(args.tri, row, nn);
        };
        auto ld = [&](const T *p) -> T {
            if constexpr (THROUGH) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            else return *p;
        };
        auto st = [&](T *p, T v) {
            if constexpr (THROUGH) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            else *p = v;
        };
        auto fetch = [&](int b) {
            const int j = b / (MF::R / RB), r0 = (b % (MF::R / RB)) * RB;
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                const int nn = ncol + j * W + MF::acc_i(r0 + r, elane);
                const T *p = Cg + (int64_t)nn * args.ldc + mrow;
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    // (not in the large fp64 tiles: their k loop is at the limit of the registers, and
                    // this change to their epilogue, like any other that was tried, costs the loop 5 %:
                    // 5000 x 3000 x 7000 3.05 -> 3.21 ms)
                    if constexpr (MASKED && THROUGH && (sizeof(T) == 4 || BM * BN <= 64 * 64)) {
                        // a load of device scope under a condition is a branch of its own that waits
                        // for its value before the next one is issued: read the tile's first element
                        // instead of a place past the edge, and let all loads of the batch fly together
                        const bool in = keep(mrow + i * W, nn);
                        const T v = ld(in ? p + i * W : Cg + (int64_t)n0 * args.ldc + m0);
                        cbuf[b & 1][r][i] = in ? v : T(0);
                    } else {
                        cbuf[b & 1][r][i] = keep(mrow + i * W, nn) ? ld(p + i * W) : T(0);
                    }
                }
            }
        };
        if (beta != T(0)) fetch(0);
#pragma unroll
        for (int b = 0; b < NBATCH; ++b) {
            const int j = b / (MF::R / RB), r0 = (b % (MF::R / RB)) * RB;
            // the next batch of C is on its way while this one is combined and stored
            if (beta != T(0) && b + 1 < NBATCH) fetch(b + 1);
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                const int nn = ncol + j * W + MF::acc_i(r0 + r, elane);
                T *p = Cg + (int64_t)nn * args.ldc + mrow;
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    // beta*c rounded, then one fused alpha*acc + that: written out, so that every
                    // instantiation of this kernel rounds alike (left to the compiler, the product that
                    // is fused into the sum is alpha*acc in one copy of this code and beta*c in another)
                    const T a = acc[i][j][r0 + r];
                    if (keep(mrow + i * W, nn))
                        st(p + i * W, (beta == T(0)) ? alpha * a : fused(alpha, a, beta * cbuf[b & 1][r][i]));
                }
            }
        }
    };
    bool through = false;
    if constexpr (SHARED) {
        through = slab_begin > 0 || slab_end < slabs_of_tile;
        if (slab_begin > 0 && !FOLLOWUP) {
            // The piece before this one is held by the workgroup before this one.  On a GPU
            // that has this launch to itself that workgroup was dispatched earlier, and it
            // raises its flag without waiting for anybody, so the wait ends.  Beside other
            // launches it may still be queued while this one holds a place it needs: the wait
            // is bounded, and a piece whose wait runs out leaves C alone, says so, and raises
            // no flag; the launch that follows this one makes up for it (see GemmArgs).
            // (the word the outcome travels in: the first padding element of an LDS row, which
            // the k loop neither reads nor writes - other wavefronts may still be in theirs)
            int *word = reinterpret_cast<int *>(lds + BM);
            if (t == 0) {
                unsigned *flag = args.sk_flags + (blockIdx.x - 1);
                long spins = 0;
                int out = 0;
                while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != args.sk_epoch) {
                    if (++spins > args.sk_spin_limit) {
                        out = 1;
                        break;
                    }
                    __builtin_amdgcn_s_sleep(8);
                }
                if (out) {
                    __hip_atomic_store(args.sk_flags + kSkMaxGroups + blockIdx.x, args.sk_epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_fetch_add(args.sk_status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                } else {
                    __hip_atomic_store(flag, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);    // as the next launch expects it
                }
                *word = out;
            }
            __syncthreads();
            if (*word != 0) return;     // (a piece that waits is its workgroup's last)
        }
    }
    if constexpr (RAGGED) {
        epilogue(std::true_type{}, std::false_type{});
    } else if constexpr (SHARED) {
        if (edge) {
            if (through) epilogue(std::true_type{}, std::true_type{});
            else epilogue(std::true_type{}, std::false_type{});
        } else {
            if (through) epilogue(std::false_type{}, std::true_type{});
            else epilogue(std::false_type{}, std::false_type{});
        }
    } else {
        // (of the triangular launches only the one over the diagonal blocks has tiles that the
        // triangle cuts; the tiles of the other lie strictly inside it)
        if (args.tri != 0 && args.tri_block != 0) {
            epilogue(std::true_type{}, std::false_type{});
        } else {
            epilogue(std::false_type{}, std::false_type{});
        }
    }
    if constexpr (SHARED) {
        if (slab_end < slabs_of_tile) {
            // every store of this piece has been acknowledged by the memory it went through to
            // before the flag is raised
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (t == 0 && !args.sk_mute)
                __hip_atomic_store(args.sk_flags + blockIdx.x, args.sk_epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    }   // pieces
}

// C <- beta*C on the m x n window: the alpha == 0 || k == 0 path of
// ulmblas/level3/gemm.tcc:52-55 (gescal, ulmblas/level1/scal.tcc:15-23).
// beta == 0 stores zeros without reading; beta == 1 is never launched.
template <typename T>
__global__ void scale_kernel(int m, int n, T beta, T *C, int64_t ldc, int tri)
{
    const int64_t total = (int64_t)m * n;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total;
         e += (int64_t)gridDim.x * blockDim.x) {
        const int64_t j = e / m, i = e - j * m;
        if (!in_triangle(tri, (int)i, (int)j)) continue;
        T *p = C + j * ldc + i;
        *p = (beta == T(0)) ? T(0) : (*p) * beta;
    }
}

}  // namespace ulmgpu
