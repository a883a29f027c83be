// Host side of libulmblas_gpu: the BLAS / CBLAS entry points of ulmBLAS's
// interface layer (interfaces/blas/F77/gemm.cc, interfaces/blas/C/gemm.cc)
// re-implemented over the HIP kernels of gemm_kernel.hip.h.  The argument
// checks, info codes, trans decoding and the row-major operand swap follow
// the reference line by line in meaning; everything below the checks is new.
#include "../../include/ulmblas_gpu.h"
#include "gemm_kernel.hip.h"
#include "internal.h"

#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <cctype>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

using namespace ulmgpu;

namespace ulmgpu {

thread_local std::string g_last_error;

bool hip_ok(hipError_t e, const char *what)
{
    if (e == hipSuccess) return true;
    g_last_error = std::string(what) + ": " + hipGetErrorString(e);
    return false;
}

// ---------------------------------------------------------------------------
// kernel variants
// ---------------------------------------------------------------------------
template <typename T>
struct Variant {
    const char *name;
    int bm, bn, bk;
    bool ragged;      // any m x n (true) or whole tiles only (false)
    int cu_slots;     // workgroups of this variant one CU holds at a time
    int wg_waves;     // wavefronts per SIMD one workgroup brings
    // The launch planner's figures for this tile, fitted by least squares to timings of launches of whole
    // tiles (a quarter of a round to eight rounds of tiles, k = 256, 1024, 4096, beta == 0 and != 0; 48
    // launches a variant, residuals 2 - 5 %): a round of c workgroups on a CU takes, per k-slab,
    // max(c x matrix-pipe cycles of the slab / eff, latency) cycles, plus per tile ovh0 + ovh1 x bytes of C
    // moved (read and written) - that in full for a workgroup alone on its CU, `company` of it otherwise.
    float eff;        // fraction of the matrix pipe's rate a full CU sustains inside the k loop
    float latency;    // cycles one k-slab takes a workgroup that has the CU to itself
    float ovh0, ovh1, company;
    float single;     // (any-shape tiles, not fitted: factor on eff for one wave per SIMD)
    // Tiles that share (fitted the same way to 50 - 120 timings a variant of launches over all of C with and
    // without shared tiles, orders 400 ... 5100): the k loop of a launch with tiles past the edge of C takes
    // `edge` times as long; a workgroup of the shared part `share_slab` times as long again per slab (no two
    // of them walk the same k at the same time, so L2 does not share their panels); folding the pieces of a
    // tile costs share_base plus share_link cycles for every piece after the first - wait, read, add,
    // write, wait for the write, one piece after the other - of which the fraction share_hidden shows when
    // whole rounds of tiles run first and the shared part's workgroups start as CUs come free.
    float edge, share_slab, share_base, share_link, share_hidden;
    int (*launch)(const GemmArgs &, T, T, bool, bool, hipStream_t);
    // the same kernel with 16-byte global loads, for 16-byte aligned A and B
    // (null for the any-shape variants)
    int (*launch_wide)(const GemmArgs &, T, T, bool, bool, hipStream_t);
    // the 16-byte-load kernel that can share tiles between workgroups along k
    // (null for variants that never do)
    int (*launch_shared)(const GemmArgs &, T, T, bool, bool, hipStream_t);
};

template <class CFG, bool RAGGED, bool TA, bool TB, bool SHARED = false, bool FOLLOWUP = false>
int launch_one(const GemmArgs &a, typename CFG::T alpha, typename CFG::T beta,
               hipStream_t stream)
{
    auto kernel = gemm_kernel<CFG, TA, TB, RAGGED, SHARED, FOLLOWUP>;
    // LDS above the 64 KiB default needs an explicit opt-in, once per kernel.
    static std::once_flag once;
    static hipError_t attr_status = hipSuccess;
    std::call_once(once, [&] {
        attr_status = hipFuncSetAttribute(
            reinterpret_cast<const void *>(kernel),
            hipFuncAttributeMaxDynamicSharedMemorySize, (int)CFG::LDS_BYTES);
    });
    HIP_TRY(attr_status);
    // every tile of the shared part is replaced by its share of the sk_groups workgroups; the launch
    // that follows up on a launch with shared tiles has one workgroup per shared tile
    const unsigned grid = FOLLOWUP
                              ? (unsigned)a.sk_tiles
                              : (unsigned)a.tiles_m * (unsigned)a.tiles_n - (SHARED ? a.sk_tiles : 0) + (SHARED ? a.sk_groups : 0);
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(CFG::NT), CFG::LDS_BYTES,
                       stream, a, alpha, beta);
    HIP_TRY(hipGetLastError());
    return ULMBLAS_GPU_OK;
}

template <class CFG, bool RAGGED>
int launch_cfg(const GemmArgs &a, typename CFG::T alpha, typename CFG::T beta,
               bool ta, bool tb, hipStream_t stream)
{
    if (!ta && !tb) return launch_one<CFG, RAGGED, false, false>(a, alpha, beta, stream);
    if (ta && !tb) return launch_one<CFG, RAGGED, true, false>(a, alpha, beta, stream);
    if (!ta && tb) return launch_one<CFG, RAGGED, false, true>(a, alpha, beta, stream);
    return launch_one<CFG, RAGGED, true, true>(a, alpha, beta, stream);
}

template <class CFG>
int launch_shared_cfg(const GemmArgs &a, typename CFG::T alpha, typename CFG::T beta,
                      bool ta, bool tb, hipStream_t stream)
{
    if (a.sk_repair) {
        if (!ta && !tb) return launch_one<CFG, false, false, false, true, true>(a, alpha, beta, stream);
        if (ta && !tb) return launch_one<CFG, false, true, false, true, true>(a, alpha, beta, stream);
        if (!ta && tb) return launch_one<CFG, false, false, true, true, true>(a, alpha, beta, stream);
        return launch_one<CFG, false, true, true, true, true>(a, alpha, beta, stream);
    }
    if (!ta && !tb) return launch_one<CFG, false, false, false, true>(a, alpha, beta, stream);
    if (ta && !tb) return launch_one<CFG, false, true, false, true>(a, alpha, beta, stream);
    if (!ta && tb) return launch_one<CFG, false, false, true, true>(a, alpha, beta, stream);
    return launch_one<CFG, false, true, true, true>(a, alpha, beta, stream);
}

#define WHOLE_VARIANT(T, BM, BN, BK, WM, WN, OCC, PF, EFF, LAT, O0, O1, CO)                    \
    {"whole_" #BM "x" #BN "x" #BK "_w" #WM "x" #WN, BM, BN, BK, false, OCC, (WM * WN + 3) / 4, EFF, LAT, O0, O1, CO, 1.0f, 1.f, 1.f, 0.f, 0.f, 1.f,  \
     &launch_cfg<Config<T, BM, BN, BK, WM, WN, OCC, PF>, false>,                              \
     &launch_cfg<Config<T, BM, BN, BK, WM, WN, OCC, PF, 16 / sizeof(T)>, false>, nullptr}
// a whole-tile variant that exists with 16-byte loads only (element-wise loads of its tile do not
// fit the registers): left out of the choice while those loads are switched off
#define WIDE_VARIANT(T, BM, BN, BK, WM, WN, OCC, PF, EFF, LAT, O0, O1, CO)                     \
    {"whole_" #BM "x" #BN "x" #BK "_w" #WM "x" #WN, BM, BN, BK, false, OCC, (WM * WN + 3) / 4, EFF, LAT, O0, O1, CO, 1.0f, 1.f, 1.f, 0.f, 0.f, 1.f,  \
     nullptr, &launch_cfg<Config<T, BM, BN, BK, WM, WN, OCC, PF, 16 / sizeof(T)>, false>, nullptr}
// a whole-tile variant that can also share tiles between workgroups along k
#define SHARING_VARIANT(T, BM, BN, BK, WM, WN, OCC, PF, EFF, LAT, O0, O1, CO, ED, SS, SB, SL, SH)                  \
    {"whole_" #BM "x" #BN "x" #BK "_w" #WM "x" #WN, BM, BN, BK, false, OCC, (WM * WN + 3) / 4, EFF, LAT, O0, O1, CO, 1.0f, ED, SS, SB, SL, SH,  \
     &launch_cfg<Config<T, BM, BN, BK, WM, WN, OCC, PF>, false>,                              \
     &launch_cfg<Config<T, BM, BN, BK, WM, WN, OCC, PF, 16 / sizeof(T)>, false>,              \
     &launch_shared_cfg<Config<T, BM, BN, BK, WM, WN, OCC, PF, 16 / sizeof(T)>>}
#define RAGGED_VARIANT(T, BM, BN, BK, WM, WN, OCC, PF, EFF, LAT)                   \
    {"ragged_" #BM "x" #BN "x" #BK "_w" #WM "x" #WN, BM, BN, BK, true, OCC, (WM * WN + 3) / 4, EFF, LAT, 6000.f, 1.f / 64.f, 0.3f, 0.95f, 1.f, 1.f, 0.f, 0.f, 1.f, \
     &launch_cfg<Config<T, BM, BN, BK, WM, WN, OCC, PF>, true>, nullptr, nullptr}

// id = index + 1.  Whole-tile variants first (the automatic choice picks among
// them), then the any-shape variants (the first of those serves the ragged
// strips and problems smaller than a tile).
const Variant<double> kVariantsD[] = {
    // (the last two numbers: the fraction of the matrix pipe's rate a CU full of this tile reaches (a
    // workgroup with one wave per SIMD alone on its CU reaches 0.95 of that), and the cycles per
    // k-slab of a workgroup alone on its CU, both from timings of whole-tile products)
    SHARING_VARIANT(double, 256, 128, 16, 4, 2, 1, 1, 0.947f, 5250.f, 7362.f, 0.0674f, 0.50f, 1.007f, 1.013f, 39140.f, 75049.f, 0.76f),
    SHARING_VARIANT(double, 128, 128, 16, 2, 2, 2, 1, 0.943f, 4397.f, 10293.f, 0.0552f, 1.00f, 1.021f, 1.161f, 4939.f, 39971.f, 0.30f),
    WHOLE_VARIANT(double, 128, 64, 16, 2, 2, 2, 1, 0.948f, 2185.f, 10325.f, 0.0558f, 1.00f),
    WHOLE_VARIANT(double, 64, 128, 16, 2, 2, 2, 1, 0.931f, 2397.f, 9942.f, 0.0500f, 1.00f),
    WHOLE_VARIANT(double, 64, 64, 16, 2, 2, 3, 2, 0.878f, 1384.f, 8021.f, 0.0561f, 1.00f),
    SHARING_VARIANT(double, 64, 64, 16, 4, 2, 2, 2, 0.909f, 1295.f, 8057.f, 0.0588f, 1.00f, 1.063f, 1.085f, 3458.f, 8958.f, 0.80f),    // 8 waves on a small tile: one workgroup fills a CU's SIMDs
    WHOLE_VARIANT(double, 32, 32, 32, 2, 2, 4, 1, 0.631f, 1275.f, 5361.f, 0.0692f, 1.00f),     // products with fewer 64 x 64 tiles than CUs
    // panels 64 wide or high (the update shapes of a blocked factorisation): one workgroup per CU
    // with two slabs on their way from HBM
    WIDE_VARIANT(double, 256, 64, 16, 4, 2, 1, 2, 0.973f, 403.f, 9890.f, 0.0590f, 0.50f),
    WIDE_VARIANT(double, 64, 256, 16, 2, 4, 1, 2, 0.944f, 4164.f, 11849.f, 0.0604f, 0.50f),
    // (element-wise masked loads: a slab takes longer to arrive)
    RAGGED_VARIANT(double, 64, 64, 16, 2, 2, 3, 2, 0.78f, 1850.f),
    RAGGED_VARIANT(double, 128, 64, 16, 2, 2, 2, 1, 0.78f, 1850.f),
};
const Variant<float> kVariantsS[] = {
    // (rates from 4096^3 and 6144^3, the small tiles' from 512^3 ... 2048^3)
    SHARING_VARIANT(float, 256, 256, 16, 4, 2, 1, 1, 0.901f, 7520.f, 8832.f, 0.0567f, 0.50f, 0.997f, 1.021f, 10476.f, 53421.f, 0.80f),
    SHARING_VARIANT(float, 256, 128, 16, 2, 2, 2, 1, 0.927f, 4519.f, 12234.f, 0.0526f, 1.00f, 1.062f, 1.010f, 18752.f, 31821.f, 0.70f),
    WHOLE_VARIANT(float, 128, 128, 16, 2, 2, 2, 2, 0.947f, 2244.f, 12272.f, 0.0576f, 1.00f),
    SHARING_VARIANT(float, 64, 64, 16, 2, 2, 4, 2, 0.784f, 918.f, 5709.f, 0.0746f, 1.00f, 1.013f, 1.118f, 941.f, 11834.f, 0.70f),
    // (the loads, not the matrix pipe, bound the any-shape kernel in single precision)
    RAGGED_VARIANT(float, 64, 64, 16, 2, 2, 3, 2, 0.45f, 2000.f),
    RAGGED_VARIANT(float, 128, 128, 16, 2, 2, 2, 1, 0.45f, 2000.f),
};
constexpr int kNumD = sizeof(kVariantsD) / sizeof(kVariantsD[0]);
constexpr int kNumS = sizeof(kVariantsS) / sizeof(kVariantsS[0]);
constexpr int kNumCUs = 256;

std::atomic<int> g_forced_d{0}, g_forced_s{0};
std::atomic<bool> g_narrow_loads{false};   // testing: never take the 16-byte-load kernels

// ---------------------------------------------------------------------------
// Tiles shared between workgroups (see GemmArgs::sk_groups).  The flags the
// workgroups of one launch raise for each other live in a device array that
// is part of the library, one row per launch in flight: launch number i uses
// row i % kSkRing and raises its flags to i + 1 (never 0), and every flag is
// put back to 0 by the workgroup that waited for it, so a row is clean when
// its launch has ended.  Launches on one stream follow one another; launches
// on different streams meet in a row only if kSkRing launches with a shared
// part are issued while one of them is still running.  A row has a second
// half in which a workgroup whose wait ran out marks itself; the launch that
// follows every launch with shared tiles reads those marks, recomputes what
// is missing and puts the row in order again.  A launch that is being
// captured into a graph shares no tile: its row and flag value would be the
// same on every replay, and replays of two graphs made from one capture may
// run at the same time.
// The status words count the waits that ran out: word 0 for launches through
// the device entry points, word 1 + i for those of host context i.
// ---------------------------------------------------------------------------
constexpr int kSkRing = 1024;
constexpr int kSkMinSlabs = 8;              // a piece of a tile is at least this many k slabs
constexpr int kSkStatusWords = 8;
static_assert(kSkStatusWords > kMaxContexts, "a status word per host context");
static __device__ unsigned g_sk_flags[kSkRing * 2 * kSkMaxGroups];
static __device__ unsigned g_sk_status[kSkStatusWords];
std::atomic<unsigned> g_sk_serial{0};
std::atomic<int> g_busy_contexts{0};        // host calls under way (each in a context of its own)
thread_local int g_status_slot = 0;         // which status word this thread's launches count in
thread_local long g_shared_launches = 0;    // launches with shared tiles this thread has made since it last asked
std::atomic<int> g_tri_way{0};              // triangular products: 0 by estimate; 1 - 3: see ULMBLAS_GPU_TEST_TRI_WAY
std::atomic<int> g_sk_max_pieces{32};       // 0: tiles are never shared
std::atomic<long> g_sk_spin_limit{1L << 20};
std::atomic<bool> g_sk_mute{false};         // testing: flags are never raised
std::atomic<int> g_whole_c{-1};             // testing: 1 = one launch over all of C wherever possible, 0 = never, -1 = by cost

constexpr int kMaxDevices = 64;
struct SkDevice {
    unsigned *flags = nullptr, *status = nullptr;
};
std::mutex g_sk_mu;
SkDevice g_sk_dev[kMaxDevices];             // where the two arrays live on each device (guarded by g_sk_mu)

// Device addresses of the flag rows and the status words on the current device;
// false (nothing set in g_last_error) when the stream is being captured or the
// addresses cannot be had: the caller then shares no tile.
bool sk_device(hipStream_t stream, SkDevice &out)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return false;
    }
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &st) != hipSuccess || st != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return false;
    }
    std::lock_guard<std::mutex> lock(g_sk_mu);
    SkDevice &d = g_sk_dev[dev];
    if (!d.flags) {
        void *f = nullptr, *w = nullptr;
        if (hipGetSymbolAddress(&f, HIP_SYMBOL(g_sk_flags)) != hipSuccess ||
            hipGetSymbolAddress(&w, HIP_SYMBOL(g_sk_status)) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        d.flags = static_cast<unsigned *>(f);
        d.status = static_cast<unsigned *>(w);
    }
    out = d;
    return true;
}

// How the tiles of a launch are dealt: `tiles` workgroup tiles of `slabs` k
// slabs each on `slots` workgroup slots of the GPU.  Whole rounds of tiles get
// a workgroup each; the tiles of the last, partial round are cut along k into
// `groups` equal runs of slabs (0: no tile is shared).
struct SharedPlan {
    int groups = 0, tiles = 0;
};
SharedPlan plan_shared(long tiles, int slabs, long slots, int max_pieces)
{
    SharedPlan p;
    const long rest = tiles % slots;
    if (max_pieces < 2 || rest == 0 || rest * 10 > slots * 9) return p;      // the last round is full, or nearly
    long groups = std::min<long>(slots, rest * slabs / kSkMinSlabs);
    groups = std::min<long>(groups, rest * max_pieces);
    groups = std::min<long>(groups, kSkMaxGroups);
    // the same number of pieces for every tile where that costs less than a fifth of the workgroups: pieces
    // that straddle two tiles make the chains of waits longer (1700^3, 217 tiles of 64 x 64: 434 workgroups
    // 0.179 ms, 512 workgroups 0.188 ms)
    if (groups >= 2 * rest && groups % rest != 0 && (groups / rest * rest) * 5 >= groups * 4) groups = groups / rest * rest;
    if (groups <= rest) return p;
    p.groups = (int)groups;
    p.tiles = (int)rest;
    return p;
}

template <typename T> struct Table;
template <> struct Table<double> {
    static const Variant<double> *v() { return kVariantsD; }
    static int count() { return kNumD; }
    static int forced() { return g_forced_d.load(); }
    static constexpr double kFlopsPerCycleCU = 128.0;   // 4 SIMDs x 2048 flop / 64 cycles
};
template <> struct Table<float> {
    static const Variant<float> *v() { return kVariantsS; }
    static int count() { return kNumS; }
    static int forced() { return g_forced_s.load(); }
    static constexpr double kFlopsPerCycleCU = 256.0;   // 4 SIMDs x 4096 flop / 64 cycles
};

template <typename T> int first_ragged_variant();

// C <- beta*C on the m x n window (beta != 1)
template <typename T>
int launch_scale(int m, int n, T beta, T *dC, int64_t ldC, hipStream_t stream, int tri)
{
    const long total = (long)m * n;
    const int threads = 256;
    const unsigned blocks = (unsigned)std::min<long>((total + threads - 1) / threads, 65536);
    hipLaunchKernelGGL(scale_kernel<T>, dim3(blocks), dim3(threads), 0, stream, m, n, beta, dC, ldC, tri);
    HIP_TRY(hipGetLastError());
    return ULMBLAS_GPU_OK;
}

// Estimated cycles of the busiest CU for `wgs` workgroup tiles of variant v,
// each walking `slabs` k-slabs.  A CU runs its share in rounds of up to
// cu_slots concurrent workgroups; a round of c of them takes, per slab, the
// matrix-pipe time of c tiles at the variant's rate but never less than what
// a workgroup alone on the CU needs for a slab (the dependent chain load ->
// LDS write -> barrier -> LDS read -> MFMA, which one workgroup cannot hide
// from itself), plus the tiles' prologue and epilogue (see Variant).
// With `share` given, the tiles of the last round are cut along k where that
// is worth it (*share then says how; otherwise it comes back empty).
template <typename T>
double estimate_cycles(const Variant<T> &v, long wgs, int slabs, bool reads_c, SharedPlan *share = nullptr, bool edges = false)
{
    const double slab_mfma = 2.0 * v.bm * v.bn * v.bk / Table<T>::kFlopsPerCycleCU;
    const double slab_latency = v.latency;
    // prologue and epilogue of a tile: launch, first slabs, C written (and read)
    const double ovh = v.ovh0 + v.ovh1 * (double)v.bm * v.bn * sizeof(T) * (reads_c ? 2 : 1);
    const long per_cu = (wgs + kNumCUs - 1) / kNumCUs;
    const double loop = edges ? v.edge : 1.0;
    auto round_cycles = [&](int c) {
        const double eff = v.eff * (c * v.wg_waves >= 2 ? 1.0 : v.single);
        return loop * slabs * std::max(c * slab_mfma / eff, slab_latency) + (c == 1 ? ovh : v.company * ovh);
    };
    const long full = per_cu / v.cu_slots;
    const int rem = (int)(per_cu % v.cu_slots);
    const double whole = full * round_cycles(v.cu_slots) + (rem ? round_cycles(rem) : 0.0);
    if (!share) return whole;
    *share = SharedPlan();
    if (!v.launch_shared || g_narrow_loads.load()) return whole;
    const long slots = (long)kNumCUs * v.cu_slots;
    // Whole rounds as ever; the shared part as the variant's figures say (see Variant).  On top: the launch
    // that follows every launch with shared tiles (11 thousand cycles when it finds nothing to do).
    const double eff = v.eff * (v.cu_slots * v.wg_waves >= 2 ? 1.0 : v.single);
    const int limit = g_sk_max_pieces.load();
    const bool forced = limit < 0;                          // testing: share whenever it can be done
    if (std::abs(limit) < 2) return whole;
    // (tiles of fewer than 24 slabs are left whole: the figures for the folds come from products with k >= 400
    // - 400^3 in two pieces a tile gains 4 - 6 % in all four transpositions -, and 5834 x 2492 x 256 cut in two
    // pieces a tile took 0.178 ms against 0.146 ms whole)
    if (!forced && slabs < 24) return whole;
    double best = whole;
    for (int cap = forced ? -limit : std::min(limit, 2); cap <= std::abs(limit); cap *= 2) {
        const SharedPlan p = plan_shared(wgs, slabs, slots, cap);
        if (p.groups == 0) continue;
        const long on_cu = (p.groups + kNumCUs - 1) / kNumCUs;
        const double run = (double)p.tiles * slabs / p.groups;
        const long pieces = (p.groups + p.tiles - 1) / p.tiles;
        const double fold = 11000.0 + v.share_base + (pieces - 1) * v.share_link * (wgs < slots ? 1.0 : v.share_hidden);
        const double cut = (wgs / slots) * round_cycles(v.cu_slots) +
                           loop * v.share_slab * run * std::max(on_cu * slab_mfma / eff, slab_latency) + fold;
        if (share->groups == 0 ? (forced || cut * 1.02 < whole) : cut < best) {
            *share = p;
            best = cut;
        }
    }
    return best;
}

// How a product is launched.
struct LaunchPlan {
    int id = 0;             // variant (0: none fits)
    bool whole_c = false;   // one launch over all of C, tiles that reach past its edges included;
                            // otherwise whole tiles in one launch and the strips in others
    SharedPlan share;       // of the main launch
    double cycles = 0;
};

// Variant `id` on an m x n x k product: the cheaper of its two ways.
template <typename T>
LaunchPlan plan_variant(int id, int m, int n, int k, bool reads_c, int64_t ldA, int64_t ldB)
{
    const Variant<T> &v = Table<T>::v()[id - 1];
    LaunchPlan best;
    if (v.ragged || (!v.launch && g_narrow_loads.load())) return best;
    // the kernel that shares tiles addresses a tile's slab with 32-bit byte offsets
    const int64_t reach = (int64_t)std::max(std::max(v.bm, v.bn), v.bk) * std::max(ldA, ldB) * (int64_t)sizeof(T);
    const bool reach_ok = reach < ((int64_t)1 << 32) - 4096;
    // (so do the whole-tile kernels with 16-byte loads: leading dimensions beyond that go to the any-shape kernel)
    if (!reach_ok && !g_narrow_loads.load()) return best;
    const bool shared_ok = v.launch_shared && !g_narrow_loads.load() && reach_ok;
    const int slabs = (k + v.bk - 1) / v.bk;
    const long tiles = (long)(m / v.bm) * (n / v.bn);
    if (tiles > 0) {
        const double rest = (double)m * n - (double)tiles * v.bm * v.bn;
        best.id = id;
        best.cycles = estimate_cycles<T>(v, tiles, slabs, reads_c, shared_ok ? &best.share : nullptr);
        // The strips (64 x 64 any-shape tiles that walk all of k, some 3000 cycles a slab whatever the strip's
        // width) run beside the whole-tile kernel on side streams, or after it when the main launch shares
        // tiles and so keeps every CU busy to the end.  What they add to the launch, from 580 timings of whole
        // tiles with and without their strips (orders 300 ... 4000 and eight oblong shapes, every whole-tile
        // variant): between a fifth and three fifths of one walk, with a spread of a third of a walk that
        // neither the number of strip workgroups nor the fill of the main launch's last round explains.
        double strips = 0.0;
        if (rest > 0) {
            const double walk = 3000.0 * ((k + 15) / 16);
            // (a tile that has its CU to itself leaves the strips only the CUs its last round leaves free: with
            // that round nine tenths full - 2900^3: 242 tiles of 256 x 128 - they cost a whole walk, 0.23 ms)
            const long slots = (long)kNumCUs * v.cu_slots;
            const double fill = tiles % slots ? (double)(tiles % slots) / slots : 1.0;
            const double beside = v.cu_slots > 1 ? 0.5 : fill > 0.85 ? 1.0 : fill > 0.5 ? 0.4 : sizeof(T) == 8 ? 0.17 : 0.25;
            // ... plus their own arithmetic, at a third of the matrix pipe's rate, where they are wide
            strips = (best.share.groups > 0 ? 1.0 : beside) * walk + 2.0 * rest * k / Table<T>::kFlopsPerCycleCU / kNumCUs / 0.3;
        }
        best.cycles += strips;
    }
    // all of C in one launch: the kernel that shares tiles also takes tiles past the edge
    // (a packet of a stored column must exist: at least 4 rows and columns)
    if (shared_ok && m >= 4 && n >= 4 && ((long)m % v.bm != 0 || (long)n % v.bn != 0)) {
        LaunchPlan all;
        all.id = id;
        all.whole_c = true;
        const long t = (long)((m + v.bm - 1) / v.bm) * ((n + v.bn - 1) / v.bn);
        all.cycles = estimate_cycles<T>(v, t, slabs, reads_c, &all.share, true);
        const int mode = g_whole_c.load();
        if (best.id == 0 || mode == 1 || (mode != 0 && all.cycles < best.cycles)) best = all;
    }
    return best;
}

// Automatic choice: the variant and way with the smallest estimate; id 0 when
// no whole-tile variant can be launched on the problem.
template <typename T>
LaunchPlan choose_plan(int m, int n, int k, bool reads_c, int64_t ldA, int64_t ldB)
{
    LaunchPlan best;
    for (int id = 1; id <= Table<T>::count(); ++id) {
        // the tiles made for panels (16-byte loads only, one workgroup per CU, two slabs in flight) stay with
        // panels no wider than their short side: elsewhere their rate is below what the panels gave
        // (1464 x 3000 x 1536: 0.29 - 0.33 ms against 0.235 ms for the 256 x 128 tile)
        const Variant<T> &v = Table<T>::v()[id - 1];
        if (!v.ragged && !v.launch && std::min(m, n) > std::min(v.bm, v.bn)) continue;
        const LaunchPlan p = plan_variant<T>(id, m, n, k, reads_c, ldA, ldB);
        // (a smaller tile has to win by 4 %: the estimate does not see that it moves more bytes per flop through
        // L2, which shows on products larger than the ones the figures were fitted to - 8192^3 with A transposed
        // went to 128 x 64 tiles at 15.6 ms where 256 x 128 take 14.9)
        const double handicap = (best.id != 0 && (long)v.bm * v.bn < (long)Table<T>::v()[best.id - 1].bm * Table<T>::v()[best.id - 1].bn) ? 1.04 : 1.0;
        if (p.id != 0 && (best.id == 0 || p.cycles * handicap < best.cycles)) best = p;
    }
    // The any-shape kernel alone over all of C: for products of a few tiles, ragged ones above all,
    // one launch of small masked tiles beats whole tiles with strips beside them and large tiles
    // cut along k (1000^3: 49 us against 96 and 130; 500^3: 26 against 117).
    const int rid = first_ragged_variant<T>();
    if (best.id != 0 && rid != 0) {
        const Variant<T> &r = Table<T>::v()[rid - 1];
        const long t = (long)((m + r.bm - 1) / r.bm) * ((n + r.bn - 1) / r.bn);
        const double alone = estimate_cycles<T>(r, t, (k + r.bk - 1) / r.bk, reads_c);
        // (up to a tile per CU: beyond that its rate depends on the transposition, which the estimate
        // does not see - 1024 x 3072 x 2048 with A transposed: 0.35 ms against 0.21 ms for shared 128 x 128 tiles)
        // (and at 1.2 times its estimate: the small tiles with 16-byte loads that take any shape in one launch
        // have caught up with it - 100^3: 9.3 us against its 11.0)
        if (t <= kNumCUs && 1.2 * alone < best.cycles) {
            best = LaunchPlan();
            best.cycles = alone;
        }
    }
    return best;
}

template <typename T>
int first_ragged_variant()
{
    for (int id = 1; id <= Table<T>::count(); ++id)
        if (Table<T>::v()[id - 1].ragged) return id;
    return 0;
}

template <typename T>
int launch_variant(int id, bool ta, bool tb, int m, int n, int k, T alpha,
                   const T *dA, int64_t ldA, const T *dB, int64_t ldB, T beta,
                   T *dC, int64_t ldC, hipStream_t stream, int tri = 0, int tri_whole = 0, int tri_block = 0,
                   const SharedPlan *share = nullptr, bool edges = false)
{
    const Variant<T> &v = Table<T>::v()[id - 1];
    GemmArgs a;
    a.m = m; a.n = n; a.k = k;
    a.tiles_m = (m + v.bm - 1) / v.bm;
    a.tiles_n = (n + v.bn - 1) / v.bn;
    a.A = dA; a.B = dB; a.C = dC;
    a.lda = ldA; a.ldb = ldB; a.ldc = ldC;
    a.tri = tri; a.tri_whole = tri_whole; a.tri_block = tri_block;
    a.sk_flags = nullptr; a.sk_status = nullptr; a.sk_epoch = 0; a.sk_mute = 0; a.sk_spin_limit = 0;
    a.sk_repair = 0;
    if (tri != 0 && !v.ragged) {
        if (tri_block > 0) {
            // the tiles of the diagonal blocks, block after block
            a.tiles_m = (m / tri_block) * (tri_block / v.bm) * (tri_block / v.bn);
            a.tiles_n = 1;
        } else {
            // only the tiles inside the triangle: ceil(T/2) folded rows of c*(T-1) tiles
            const int t = m / v.bm, c = v.bm / v.bn;
            a.tiles_m = (t + 1) / 2;
            a.tiles_n = c * (t - 1);
        }
    }
    // 16-byte loads wherever the variant has them: the hardware carries them out at any
    // element-aligned address, so odd leading dimensions and offsets take them too
    const bool wide = v.launch_wide && !g_narrow_loads.load();
    a.sk_groups = a.sk_tiles = 0;
    // (of the triangular launches the one over the whole tiles inside the triangle may share tiles: its
    // grid is a rectangle of tiles like any other as long as no tile of it is left out, see the kernel)
    const bool tri_shares = tri != 0 && tri_block == 0 && !edges && (m / v.bm) % 2 == 0;
    if (wide && v.launch_shared && (tri == 0 || tri_shares) && !v.ragged && ((share && share->groups > 0) || edges)) {
        // the kernel that shares tiles between workgroups and takes tiles that reach past the edges of C
        // (not beside another host call: each launch is cut for a GPU it has to itself, and workgroups
        // that wait for workgroups which other launches keep off the GPU hold everybody up)
        if (share && share->groups > 0 && g_busy_contexts.load() <= 1) {
            SkDevice d;
            if (sk_device(stream, d)) {
                const unsigned serial = g_sk_serial.fetch_add(1);
                a.sk_groups = share->groups;
                a.sk_tiles = share->tiles;
                a.sk_flags = d.flags + (size_t)(serial % kSkRing) * 2 * kSkMaxGroups;
                a.sk_epoch = serial + 1 ? serial + 1 : 1;
                a.sk_mute = g_sk_mute.load() ? 1u : 0u;
                a.sk_spin_limit = g_sk_spin_limit.load();
                a.sk_status = d.status + g_status_slot;
            }
        }
        int rc = v.launch_shared(a, alpha, beta, ta, tb, stream);
        if (rc || a.sk_groups == 0) return rc;
        // the launch that follows up: recomputes the rest of every shared tile one of whose pieces
        // gave up its wait (none, as a rule: its workgroups look at a few words and end)
        ++g_shared_launches;
        a.sk_repair = 1;
        return v.launch_shared(a, alpha, beta, ta, tb, stream);
    }
    if (edges) {
        g_last_error = "internal: this variant cannot take tiles past the edge of C";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    if (!wide && !v.launch) {
        g_last_error = "internal: this variant has no kernel with element-wise loads";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    return (wide ? v.launch_wide : v.launch)(a, alpha, beta, ta, tb, stream);
}

// Two side streams per caller stream, so that the ragged strips of a product
// run next to its whole-tile kernel instead of after it: fork from the
// caller's stream with an event, join back with one event per strip.  Keyed
// by the caller's stream: products on different streams never meet on a side
// stream, and a capture on one caller stream (which draws that stream's side
// streams into the capture) leaves the side streams of the others alone.
// ulmblas_gpu_release() destroys them.
struct SideStreams {
    hipStream_t s[2] = {nullptr, nullptr};
    hipEvent_t fork = nullptr, join[2] = {nullptr, nullptr};
    bool ok = false;
    void create()
    {
        ok = hipStreamCreateWithFlags(&s[0], hipStreamNonBlocking) == hipSuccess &&
             hipStreamCreateWithFlags(&s[1], hipStreamNonBlocking) == hipSuccess &&
             hipEventCreateWithFlags(&fork, hipEventDisableTiming) == hipSuccess &&
             hipEventCreateWithFlags(&join[0], hipEventDisableTiming) == hipSuccess &&
             hipEventCreateWithFlags(&join[1], hipEventDisableTiming) == hipSuccess;
        if (!ok) (void)hipGetLastError();
    }
    void destroy()
    {
        for (hipStream_t &x : s) {
            if (x) (void)hipStreamDestroy(x);
            x = nullptr;
        }
        if (fork) (void)hipEventDestroy(fork);
        fork = nullptr;
        for (hipEvent_t &e : join) {
            if (e) (void)hipEventDestroy(e);
            e = nullptr;
        }
        ok = false;
    }
};
std::mutex g_side_mu;
std::condition_variable g_side_cv;
std::map<hipStream_t, SideStreams> g_side;      // guarded by g_side_mu; entries stay put once made
int g_side_users = 0;                           // calls that hold a pointer into g_side (guarded by g_side_mu)
thread_local int g_inline_strips = 0;           // > 0: strips go to the caller's stream, nothing is created

// Holds the side streams of a caller's stream for as long as a call records and waits on them:
// ulmblas_gpu_release(), which destroys them, waits until nobody does.
class SideUse {
public:
    explicit SideUse(hipStream_t stream, bool wanted);
    ~SideUse();
    SideUse(const SideUse &) = delete;
    SideUse &operator=(const SideUse &) = delete;
    SideStreams *get() const { return side_; }

private:
    SideStreams *side_ = nullptr;
};

// The side streams of `stream`, made on first use; null when they cannot be
// had, when the calling thread asked for none (InlineStrips), or when the
// caller's stream is being captured and its side streams do not exist yet
// (creating streams in the middle of a capture is left alone).
SideStreams *side_streams_of_locked(hipStream_t stream)
{
    if (g_inline_strips > 0) return nullptr;
    auto it = g_side.find(stream);
    if (it == g_side.end()) {
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &st) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        if (st != hipStreamCaptureStatusNone) return nullptr;
        if (g_side.size() >= 64) return nullptr;      // a caller that makes streams without end gets no more
        it = g_side.emplace(stream, SideStreams()).first;
        it->second.create();
    }
    return it->second.ok ? &it->second : nullptr;
}

SideUse::SideUse(hipStream_t stream, bool wanted)
{
    if (!wanted) return;
    std::lock_guard<std::mutex> lock(g_side_mu);
    side_ = side_streams_of_locked(stream);
    if (side_) ++g_side_users;
}

SideUse::~SideUse()
{
    if (!side_) return;
    {
        std::lock_guard<std::mutex> lock(g_side_mu);
        --g_side_users;
    }
    g_side_cv.notify_all();
}

void release_side_streams()
{
    std::unique_lock<std::mutex> lock(g_side_mu);
    g_side_cv.wait(lock, [] { return g_side_users == 0; });
    for (auto &kv : g_side) kv.second.destroy();
    g_side.clear();
}

InlineStrips::InlineStrips() { ++g_inline_strips; }
InlineStrips::~InlineStrips() { --g_inline_strips; }

template <typename T>
int gemm_device(bool ta, bool tb, int m, int n, int k, T alpha, const T *dA,
                int ldA, const T *dB, int ldB, T beta, T *dC, int ldC,
                hipStream_t stream)
{
    const int rowsA = ta ? k : m, rowsB = tb ? n : k;
    if (m < 0 || n < 0 || k < 0 || ldA < std::max(1, rowsA) ||
        ldB < std::max(1, rowsB) || ldC < std::max(1, m)) {
        g_last_error = "invalid size or leading dimension";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    if (m == 0 || n == 0) return ULMBLAS_GPU_OK;
    if (!dC || ((alpha != T(0) && k > 0) && (!dA || !dB))) {
        g_last_error = "null operand";
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }

    // ulmblas/level3/gemm.tcc:52-55
    if (alpha == T(0) || k == 0) {
        if (beta == T(1)) return ULMBLAS_GPU_OK;
        return launch_scale<T>(m, n, beta, dC, ldC, stream);
    }

    const int forced = Table<T>::forced();
    const int ragged_id = first_ragged_variant<T>();
    LaunchPlan plan;
    if (forced > 0 && forced <= Table<T>::count()) {
        plan = plan_variant<T>(forced, m, n, k, beta != T(0), ldA, ldB);
        if (plan.id == 0) {             // an any-shape variant, or a whole-tile one with no tile in the problem
            return launch_variant<T>(Table<T>::v()[forced - 1].ragged ? forced : ragged_id, ta, tb, m, n, k, alpha, dA,
                                     ldA, dB, ldB, beta, dC, ldC, stream);
        }
    } else {
        plan = choose_plan<T>(m, n, k, beta != T(0), ldA, ldB);
        if (plan.id == 0) {
            return launch_variant<T>(ragged_id, ta, tb, m, n, k, alpha, dA, ldA, dB, ldB, beta, dC, ldC, stream);
        }
    }
    const int id = plan.id;
    const Variant<T> &v = Table<T>::v()[id - 1];
    if (plan.whole_c) {
        return launch_variant<T>(id, ta, tb, m, n, k, alpha, dA, ldA, dB, ldB, beta, dC, ldC, stream, 0, 0, 0,
                                 &plan.share, true);
    }
    const int m_whole = (m / v.bm) * v.bm, n_whole = (n / v.bn) * v.bn;

    // whole tiles on the caller's stream; the right strip (all rows) and the
    // bottom strip beside it on the side streams
    const int64_t a_sx = ta ? ldA : 1;        // distance between rows of op(A)
    const int64_t b_sx = tb ? 1 : ldB;        // distance between columns of op(B)
    const bool right = n > n_whole, bottom = m > m_whole;
    // A launch that shares tiles keeps every CU busy from start to end: strips beside it would only
    // take matrix-pipe time from workgroups that others wait for, so there they follow on the same stream.
    const bool fills_gpu = plan.share.groups > 0;
    const SideUse side_use(stream, (right || bottom) && !fills_gpu);
    SideStreams *side = side_use.get();
    const bool forked = side != nullptr;
    if (forked) {
        HIP_TRY(hipEventRecord(side->fork, stream));
        if (right) HIP_TRY(hipStreamWaitEvent(side->s[0], side->fork, 0));
        if (bottom) HIP_TRY(hipStreamWaitEvent(side->s[1], side->fork, 0));
    }
    int rc = launch_variant<T>(id, ta, tb, m_whole, n_whole, k, alpha, dA, ldA, dB, ldB, beta, dC, ldC, stream, 0, 0, 0,
                               &plan.share);
    if (rc) return rc;
    if (right) {
        hipStream_t s = forked ? side->s[0] : stream;
        rc = launch_variant<T>(ragged_id, ta, tb, m, n - n_whole, k, alpha, dA, ldA, dB + n_whole * b_sx, ldB, beta,
                               dC + (int64_t)n_whole * ldC, ldC, s);
        if (rc) return rc;
        if (forked) {
            HIP_TRY(hipEventRecord(side->join[0], s));
            HIP_TRY(hipStreamWaitEvent(stream, side->join[0], 0));
        }
    }
    if (bottom) {
        hipStream_t s = forked ? side->s[1] : stream;
        rc = launch_variant<T>(ragged_id, ta, tb, m - m_whole, n_whole, k, alpha, dA + m_whole * a_sx, ldA, dB, ldB,
                               beta, dC + m_whole, ldC, s);
        if (rc) return rc;
        if (forked) {
            HIP_TRY(hipEventRecord(side->join[1], s));
            HIP_TRY(hipStreamWaitEvent(stream, side->join[1], 0));
        }
    }
    return ULMBLAS_GPU_OK;
}

// One triangle (tri = +1: row >= column, -1: row <= column) of the n x n
// block C <- alpha*op(A)*op(B) + beta*C, diagonal included; the other triangle
// of C is neither read nor written.  Tiles off the triangle exit at once.
template <typename T>
int gemm_tri_device(int tri, bool ta, bool tb, int n, int k, T alpha, const T *dA, int ldA, const T *dB, int ldB,
                    T beta, T *dC, int ldC, hipStream_t stream)
{
    if (n <= 0) return ULMBLAS_GPU_OK;
    if (alpha == T(0) || k == 0) {
        if (beta == T(1)) return ULMBLAS_GPU_OK;
        return launch_scale<T>(n, n, beta, dC, ldC, stream, tri);
    }
    // the last any-shape variant has the larger tile
    int ragged_id = 0;
    for (int i = 0; i < Table<T>::count(); ++i) {
        if (Table<T>::v()[i].ragged) ragged_id = i + 1;
    }
    // Whole tiles strictly inside the triangle go to the first whole-tile
    // variant, over the leading square of t blocks of order `block` (its tile
    // edges divide it); the blocks on the diagonal of that square go to a
    // small whole-tile variant with masked stores; the rows (columns, for the
    // upper triangle) beyond the square are a plain product of their own, and
    // the triangle at their end goes to the any-shape kernel.
    int diag_id = 0;        // the whole-tile variant with 64 x 64 tiles that brings most waves
    for (int i = 0; i < Table<T>::count(); ++i) {
        const Variant<T> &d = Table<T>::v()[i];
        if (!d.ragged && d.bm == 64 && d.bn == 64 && d.bk == 16 &&
            (diag_id == 0 || d.wg_waves > Table<T>::v()[diag_id - 1].wg_waves)) diag_id = i + 1;
    }
    // the tiles the main launch may take: the two largest (the second for short k, where the
    // largest, alone on its CU, has nothing to run beside its epilogue)
    auto fits = [&](int wid) {
        if (wid > Table<T>::count()) return false;
        const Variant<T> &w = Table<T>::v()[wid - 1];
        // (the whole-tile kernels address a tile's slab with 32-bit byte offsets)
        const int64_t span = (int64_t)std::max(std::max(w.bm, w.bn), w.bk) * std::max(ldA, ldB) * (int64_t)sizeof(T);
        return !w.ragged && w.bm % w.bn == 0 && w.bm % 64 == 0 && n / w.bm >= 2 && span < ((int64_t)1 << 32) - 4096;
    };
    const bool split = Table<T>::forced() == 0 && diag_id != 0 && fits(1);
    if (!split) {
        return launch_variant<T>(ragged_id, ta, tb, n, n, k, alpha, dA, ldA, dB, ldB, beta, dC, ldC, stream, tri);
    }
    const bool reads_c = beta != T(0);
    // The price of a square of t blocks with what lies beyond it.  The main launch shares the tiles
    // of its last round like a plain product, which its folded grid allows for an even t only.
    struct Way {
        int wid = 0, t = 0;
        SharedPlan share;
        double cycles = 0;
    };
    auto price = [&](int wid, int t) {
        const Variant<T> &w = Table<T>::v()[wid - 1];
        Way way;
        way.wid = wid;
        way.t = t;
        const int block = w.bm, slabs = (k + w.bk - 1) / w.bk;
        const int c = w.bm / w.bn, per_block = (block / 64) * (block / 64 + 1) / 2;
        const long tiles = (long)((t + 1) / 2) * c * (t - 1);
        const int64_t reach = (int64_t)std::max(std::max(w.bm, w.bn), w.bk) * std::max(ldA, ldB) * (int64_t)sizeof(T);
        const bool may_share = t % 2 == 0 && w.launch_shared && reach < ((int64_t)1 << 32) - 4096;
        way.cycles = estimate_cycles<T>(w, tiles, slabs, reads_c, may_share ? &way.share : nullptr) +
                     estimate_cycles<T>(Table<T>::v()[diag_id - 1], (long)t * per_block, slabs, reads_c);
        const int rest = n - t * block;
        if (rest > 0) {
            way.cycles += tri > 0 ? choose_plan<T>(rest, t * block, k, reads_c, ldA, ldB).cycles
                                  : choose_plan<T>(t * block, rest, k, reads_c, ldA, ldB).cycles;
        }
        return way;
    };
    // (the test switch: 1 / 2 the largest tile with all whole blocks / an even number of them, 4 / 5 the
    // second tile likewise, 3 the any-shape kernel alone)
    const int forced_way = g_tri_way.load();
    Way way;
    for (int wid = 1; wid <= 2; ++wid) {
        if (!fits(wid) || (forced_way != 0 && forced_way != 3 && (forced_way >= 4) != (wid == 2))) continue;
        const bool all_blocks = forced_way == 1 || forced_way == 4, even_blocks = forced_way == 2 || forced_way == 5;
        const int t = n / Table<T>::v()[wid - 1].bm;
        Way cand = price(wid, t);
        if (t % 2 == 1 && t >= 3 && !all_blocks) {
            const Way even = price(wid, t - 1);
            if (even.cycles < cand.cycles || even_blocks) cand = even;
        }
        if (way.wid == 0 || cand.cycles < way.cycles) way = cand;
    }
    if (way.wid == 0) way = price(1, n / Table<T>::v()[0].bm);        // (a forced way that does not fit)
    const int block = Table<T>::v()[way.wid - 1].bm;
    // The any-shape kernel alone over the triangle: small orders, where a few large tiles walk all
    // of k with most CUs idle (n = k = 1000, fp64: 0.33 ms split against 0.05 ms for all of A*A').
    {
        const Variant<T> &r = Table<T>::v()[first_ragged_variant<T>() - 1];
        const long tr = (n + r.bm - 1) / r.bm, tc = (n + r.bn - 1) / r.bn;
        const long live = (tr * tc + std::min(tr, tc)) / 2;
        // (its rate over several rounds is below the estimate's, and far below it where it reads a
        // transposed A element by element along k: order 3072, fp64, 0.83 ms / 1.52 ms for A*A' / A'*A
        // against 0.54 ms split; so only up to three tiles per CU, and A'*A at 1.6 times the price)
        const double alone = estimate_cycles<T>(r, live, (k + r.bk - 1) / r.bk, reads_c) * (ta ? 1.6 : 1.0);
        if (forced_way == 0 ? (live <= 3 * kNumCUs && alone < way.cycles) : forced_way == 3) {
            return launch_variant<T>(first_ragged_variant<T>(), ta, tb, n, n, k, alpha, dA, ldA, dB, ldB, beta, dC, ldC,
                                     stream, tri);
        }
    }
    const int n_whole = way.t * block, rest = n - n_whole;
    const int64_t a_sx = ta ? ldA : 1;        // distance between rows of op(A)
    const int64_t b_sx = tb ? 1 : ldB;        // distance between columns of op(B)
    // The triangle at the end walks all of k in a handful of workgroups: on a side stream, beside
    // everything else.  The rest on the caller's stream, one launch after the other: side by side
    // the masked workgroups take matrix-pipe time from the whole tiles on every CU they share,
    // which costs more than the idle CUs at the end of either launch.
    const SideUse side_use(stream, rest > 0);
    SideStreams *side = side_use.get();
    if (rest > 0) {
        hipStream_t s = side ? side->s[0] : stream;
        if (side) {
            HIP_TRY(hipEventRecord(side->fork, stream));
            HIP_TRY(hipStreamWaitEvent(s, side->fork, 0));
        }
        int rc = launch_variant<T>(first_ragged_variant<T>(), ta, tb, rest, rest, k, alpha, dA + n_whole * a_sx, ldA,
                                   dB + n_whole * b_sx, ldB, beta, dC + (int64_t)n_whole * ldC + n_whole, ldC, s, tri);
        if (rc) return rc;
    }
    int rc = launch_variant<T>(way.wid, ta, tb, n_whole, n_whole, k, alpha, dA, ldA, dB, ldB, beta, dC, ldC, stream, tri,
                               0, 0, &way.share);
    if (rc) return rc;
    rc = launch_variant<T>(diag_id, ta, tb, n_whole, n_whole, k, alpha, dA, ldA, dB, ldB, beta, dC, ldC, stream, tri,
                           n_whole, block);
    if (rc || rest == 0) return rc;
    rc = tri > 0 ? gemm_device<T>(ta, tb, rest, n_whole, k, alpha, dA + n_whole * a_sx, ldA, dB, ldB, beta,
                                  dC + n_whole, ldC, stream)
                 : gemm_device<T>(ta, tb, n_whole, rest, k, alpha, dA, ldA, dB + n_whole * b_sx, ldB, beta,
                                  dC + (int64_t)n_whole * ldC, ldC, stream);
    if (rc) return rc;
    if (side) {
        // (the product above may have used the side stream after the triangle: this covers both)
        HIP_TRY(hipEventRecord(side->join[0], side->s[0]));
        HIP_TRY(hipStreamWaitEvent(stream, side->join[0], 0));
    }
    return ULMBLAS_GPU_OK;
}

// ---------------------------------------------------------------------------
// host-pointer path: device operand buffers cached between calls (the role
// of the static MemoryPool in ulmblas/level3/gemm.tcc:50,57-58,85-86)
// ---------------------------------------------------------------------------
std::atomic<long> g_host_allocs{0}, g_fail_allocs{0};
std::atomic<int> g_host_head{1};            // large host products: a head of op(B) ahead of A (0: never, 2: also
                                            // where it is not expected to pay)
thread_local int g_last_status = ULMBLAS_GPU_OK;
thread_local unsigned g_recovered = 0;      // waits that ran out (and were made up for) in this thread's last host call

namespace {
std::mutex g_ctx_mu;
std::condition_variable g_ctx_cv;
HostContext *g_ctxs[kMaxContexts];          // made on demand, never destroyed: no HIP calls at exit
bool g_ctx_busy[kMaxContexts];
thread_local int g_ctx_hint = 0;            // the context this thread had last
}  // namespace

ContextLease::ContextLease()
{
    std::unique_lock<std::mutex> lock(g_ctx_mu);
    for (;;) {
        int pick = -1;
        if (g_ctxs[g_ctx_hint] && !g_ctx_busy[g_ctx_hint]) pick = g_ctx_hint;
        for (int i = 0; pick < 0 && i < kMaxContexts; ++i)
            if (g_ctxs[i] && !g_ctx_busy[i]) pick = i;
        for (int i = 0; pick < 0 && i < kMaxContexts; ++i) {
            if (!g_ctxs[i]) {
                g_ctxs[i] = new HostContext;
                pick = i;
            }
        }
        if (pick >= 0) {
            g_ctx_busy[pick] = true;
            g_ctx_hint = index_ = pick;
            c_ = g_ctxs[pick];
            g_busy_contexts.fetch_add(1);
            g_status_slot = 1 + pick;
            g_shared_launches = 0;
            return;
        }
        g_ctx_cv.wait(lock);
    }
}

// How many waits of workgroups for one another ran out in launches that counted in status word
// `slot` of the current device; the count is cleared.  Only called when nothing that counts
// there is still running.
unsigned take_status_word(int slot)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return 0;
    }
    SkDevice d;
    {
        std::lock_guard<std::mutex> lock(g_sk_mu);
        d = g_sk_dev[dev];
    }
    unsigned word = 0;
    if (!d.status || hipMemcpy(&word, d.status + slot, sizeof(word), hipMemcpyDeviceToHost) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    if (word != 0 && hipMemset(d.status + slot, 0, sizeof(word)) != hipSuccess) (void)hipGetLastError();
    return word;
}

ContextLease::~ContextLease()
{
    // (the call is over: whatever it launched has run, or has been waited for after a failure)
    if (g_shared_launches > 0) g_recovered += take_status_word(g_status_slot);
    g_shared_launches = 0;
    g_status_slot = 0;
    g_busy_contexts.fetch_sub(1);
    {
        std::lock_guard<std::mutex> lock(g_ctx_mu);
        g_ctx_busy[index_] = false;
    }
    g_ctx_cv.notify_all();
}

void report_host_status(const char *routine, int status, HostContext *c)
{
    g_last_status = status;
    const unsigned recovered = g_recovered;
    g_recovered = 0;
    if (status == ULMBLAS_GPU_OK) {
        if (recovered > 0) {
            const std::string text = std::to_string(recovered) + " wait(s) of workgroups that shared a tile ran out; what "
                                     "they would have added was computed afterwards: the result is complete, the call took longer";
            ulmblas_gpu_error_hook(routine, ULMBLAS_GPU_RECOVERED, text.c_str());
        }
        return;
    }
    if (c) c->drain();
    ulmblas_gpu_error_hook(routine, status, g_last_error.c_str());
}

// Copy the rows x cols window of a column-major host matrix (leading
// dimension ld) to / from a compact device matrix (leading dimension rows).
template <typename T>
int copy_window(void *dst, size_t dpitch, const void *src, size_t spitch,
                int rows, int cols, hipMemcpyKind kind, hipStream_t stream)
{
    const size_t width = (size_t)rows * sizeof(T);
    if (rows == 0 || cols == 0) return ULMBLAS_GPU_OK;
    if (dpitch == width && spitch == width) {
        HIP_TRY(hipMemcpyAsync(dst, src, width * cols, kind, stream));
    } else {
        HIP_TRY(hipMemcpy2DAsync(dst, dpitch, src, spitch, width, cols, kind, stream));
    }
    return ULMBLAS_GPU_OK;
}

// The plain path: whole operands through the runtime's own staging, one stream.
template <typename T>
int gemm_host_plain(HostContext &c, bool ta, bool tb, int m, int n, int k, T alpha,
                    const T *A, int ldA, const T *B, int ldB, T beta, T *C, int ldC,
                    bool scale_only, T *dA, int dldA, T *dB, int dldB, T *dC, int dldC)
{
    int rc;
    const int rowsA = ta ? k : m, colsA = ta ? m : k;
    const int rowsB = tb ? n : k, colsB = tb ? k : n;
    if (!scale_only) {
        if ((rc = copy_window<T>(dA, (size_t)dldA * sizeof(T), A, (size_t)ldA * sizeof(T),
                                 rowsA, colsA, hipMemcpyHostToDevice, c.stream))) return rc;
        if ((rc = copy_window<T>(dB, (size_t)dldB * sizeof(T), B, (size_t)ldB * sizeof(T),
                                 rowsB, colsB, hipMemcpyHostToDevice, c.stream))) return rc;
    }
    if (beta != T(0)) {   // beta == 0: C is never read, not even copied
        if ((rc = copy_window<T>(dC, (size_t)dldC * sizeof(T), C, (size_t)ldC * sizeof(T),
                                 m, n, hipMemcpyHostToDevice, c.stream))) return rc;
    }
    if ((rc = gemm_device<T>(ta, tb, m, n, k, alpha, dA, dldA, dB, dldB, beta,
                             dC, dldC, c.stream))) return rc;
    if ((rc = copy_window<T>(C, (size_t)ldC * sizeof(T), dC, (size_t)dldC * sizeof(T),
                             m, n, hipMemcpyDeviceToHost, c.stream))) return rc;
    HIP_TRY(hipStreamSynchronize(c.stream));
    return ULMBLAS_GPU_OK;
}

template <typename T>
int gemm_host_pipelined(HostContext &c, bool ta, bool tb, int m, int n, int k, T alpha,
                        const T *A, int ldA, const T *B, int ldB, T beta, T *C, int ldC,
                        T *dA, int dldA, T *dB, int dldB, T *dC, int dldC)
{
    int rc;
    const int rowsA = ta ? k : m, colsA = ta ? m : k;
    // panels of C: wide enough to keep the GPU busy (>= 4M elements), at most 32 of them
    int panels = (int)std::min<long>(32, std::max<long>(1, ((long)m * n) / (4L << 20)));
    int nb = ((n + panels - 1) / panels + 255) / 256 * 256;
    panels = (n + nb - 1) / nb;

    const hipStream_t ks = c.stream;
    // One column panel of C: its part of op(B) (and of C) up, its product, its result on the way back.
    // The first `head` panels are treated as one wide panel whose product is spread over the arrival of A.
    int next_event = 0;
    Pipeline<T> pipe(c);
    pipe.set_free_out(c.out_ring.count());
    pipe.set_fine(panels == 1);         // nothing else overlaps the transfers of a single panel
    auto upload_columns = [&](int j0, int nj) -> int {
        int r;
        if (!tb) {      // columns j0.. of the stored k x n matrix
            r = pipe.upload(B + (size_t)j0 * ldB, ldB, dB + (size_t)j0 * dldB, dldB, k, nj);
        } else {        // rows j0.. of the stored n x k matrix, on the device a compact nj x k matrix of their
                        // own (a copy into a window of a wider matrix is not one transfer)
            r = pipe.upload(B + j0, ldB, dB + (size_t)j0 * k, nj, nj, k);
        }
        if (r) return r;
        if (beta != T(0)) r = pipe.upload(C + (size_t)j0 * ldC, ldC, dC + (size_t)j0 * dldC, dldC, m, nj);
        return r;
    };
    auto uploaded_so_far = [&]() -> int {       // the kernels queued next wait for every upload queued so far
        hipEvent_t e = c.events[next_event++];
        HIP_TRY(hipEventRecord(e, c.h2d));
        HIP_TRY(hipStreamWaitEvent(ks, e, 0));
        return ULMBLAS_GPU_OK;
    };
    auto send_back = [&](int j0, int nj) -> int {
        hipEvent_t computed = c.events[next_event++];
        HIP_TRY(hipEventRecord(computed, ks));
        pipe.want_download(dC + (size_t)j0 * dldC, C + (size_t)j0 * ldC, ldC, m, nj, computed);
        return pipe.pump(false);
    };

    // With A up first nothing is computed for as long as A travels.  So a head of op(B)'s columns
    // goes first, and A follows in panels of its stored columns, each multiplied into the head of C
    // as it lands: for op(A) = A these are runs of k (the head of C accumulates over them, beta for
    // the first and 1 for the others, as ulmblas/level3/gemm.tcc:60-83 does with its own runs of
    // k), for op(A) = A' runs of rows of C.  The head is sized so that its products are over when
    // A is up; the columns after it go panel by panel as before, now against all of A.
    int head = 0, a_panels = 1;
    // (measured, 8192^3: 29.0 -> 25.9 ms; with beta != 0 the uploads alone take longer than everything
    // else and nothing is gained, and below some 200 MB of A the coarser pipeline costs more than
    // the wait for A; the switch's value 2 lifts both conditions for the tests)
    const int mode = g_host_head.load();
    const long a_bytes = (long)rowsA * colsA * (long)sizeof(T);
    if (mode > 1 ? panels >= 3 : (mode == 1 && panels >= 4 && beta == T(0) && a_bytes >= (192L << 20))) {
        // (A of 8192^2 in 8, 10, 16, 24, 32 panels: 26.2, 26.3, 25.9, 25.9, 26.3 ms)
        a_panels = (int)std::min<long>(16, std::max<long>(mode > 1 ? 2 : 1, a_bytes / (32L << 20)));
        // products of the head per second against bytes of A per second: about 4600 columns
        // (8192^3, head of 512 ... 5120 columns: 28.9, 28.5, 27.6, 27.2, 26.4, 25.9, 26.5, 27.4, 28.7, 30.4 ms)
        const long want = std::min<long>(4608, (long)n * 3 / 8);
        head = (int)std::min<long>(panels - 2, (want + nb / 2) / nb);
        if (a_panels < 2 || head < 1) head = 0;
    }
    if ((rc = c.ensure_events(2 * (size_t)panels + (size_t)a_panels + 4))) return rc;
    if (head > 0) {
        const int n1 = head * nb;
        if ((rc = upload_columns(0, n1))) return rc;
        const int step = ((colsA + a_panels - 1) / a_panels + 255) / 256 * 256;
        for (int c0 = 0; c0 < colsA; c0 += step) {
            const int nc = std::min(step, colsA - c0);
            if ((rc = pipe.upload(A + (size_t)c0 * ldA, ldA, dA + (size_t)c0 * dldA, dldA, rowsA, nc))) return rc;
            if ((rc = uploaded_so_far())) return rc;
            const int ldB1 = tb ? n1 : dldB;        // the head of op(B) on the device
            if (!ta) {      // columns c0.. of A meet rows c0.. of op(B)
                const T *dBp = tb ? dB + (size_t)c0 * ldB1 : dB + c0;
                rc = gemm_device<T>(ta, tb, m, n1, nc, alpha, dA + (size_t)c0 * dldA, dldA, dBp, ldB1,
                                    c0 == 0 ? beta : T(1), dC, dldC, ks);
            } else {        // columns c0.. of the stored A are rows c0.. of op(A) and of C
                rc = gemm_device<T>(ta, tb, nc, n1, k, alpha, dA + (size_t)c0 * dldA, dldA, dB, ldB1, beta, dC + c0,
                                    dldC, ks);
            }
            if (rc) return rc;
            if ((rc = pipe.pump(false))) return rc;
        }
        if ((rc = send_back(0, n1))) return rc;
    } else {
        if ((rc = pipe.upload(A, ldA, dA, dldA, rowsA, colsA))) return rc;
    }
    for (int p = head; p < panels; ++p) {
        const int j0 = p * nb, nj = std::min(nb, n - j0);
        if ((rc = upload_columns(j0, nj))) return rc;
        if ((rc = uploaded_so_far())) return rc;
        const T *dBp = tb ? dB + (size_t)j0 * k : dB + (size_t)j0 * dldB;
        if ((rc = gemm_device<T>(ta, tb, m, nj, k, alpha, dA, dldA, dBp, tb ? nj : dldB, beta,
                                 dC + (size_t)j0 * dldC, dldC, ks))) return rc;
        if ((rc = send_back(j0, nj))) return rc;
    }
    if ((rc = pipe.pump(true))) return rc;
    HIP_TRY(hipStreamSynchronize(c.d2h));
    HIP_TRY(hipStreamSynchronize(c.h2d));
    HIP_TRY(hipStreamSynchronize(ks));
    return ULMBLAS_GPU_OK;
}

template <typename T>
int gemm_host(HostContext &c, bool ta, bool tb, int m, int n, int k, T alpha, const T *A,
              int ldA, const T *B, int ldB, T beta, T *C, int ldC)
{
    if (m <= 0 || n <= 0) return ULMBLAS_GPU_OK;
    const bool scale_only = (alpha == T(0) || k <= 0);
    if (scale_only && beta == T(1)) return ULMBLAS_GPU_OK;   // C untouched

    int rc = c.ensure_stream();
    if (rc) return rc;

    const int rowsA = ta ? k : m, colsA = ta ? m : k;
    const int rowsB = tb ? n : k, colsB = tb ? k : n;
    const int dldA = std::max(1, rowsA), dldB = std::max(1, rowsB), dldC = m;

    if ((rc = c.reserve(2, (size_t)dldC * n * sizeof(T)))) return rc;
    T *dC = static_cast<T *>(c.buf[2]);
    T *dA = nullptr, *dB = nullptr;
    if (!scale_only) {
        if ((rc = c.reserve(0, (size_t)dldA * colsA * sizeof(T)))) return rc;
        if ((rc = c.reserve(1, (size_t)dldB * colsB * sizeof(T)))) return rc;
        dA = static_cast<T *>(c.buf[0]);
        dB = static_cast<T *>(c.buf[1]);
    }

    // Large products take the pipelined path: worth it once the operands are
    // tens of MiB; a single column must fit one pinned chunk.
    const size_t bytes = ((size_t)rowsA * colsA + (size_t)rowsB * colsB + (size_t)m * n) * sizeof(T);
    const size_t longest_col = (size_t)std::max(std::max(rowsA, tb ? k : rowsB), m) * sizeof(T);
    if (!scale_only && bytes >= ((size_t)16 << 20) && longest_col <= PinnedRing::kChunkBytes &&
        c.ensure_pipeline()) {
        return gemm_host_pipelined<T>(c, ta, tb, m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC,
                                      dA, dldA, dB, dldB, dC, dldC);
    }
    return gemm_host_plain<T>(c, ta, tb, m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC, scale_only,
                              dA, dldA, dB, dldB, dC, dldC);
}

template <typename T>
void gemm_host_report(const char *rout, bool ta, bool tb, int m, int n, int k,
                      T alpha, const T *A, int ldA, const T *B, int ldB,
                      T beta, T *C, int ldC)
{
    if (m <= 0 || n <= 0 || ((alpha == T(0) || k <= 0) && beta == T(1))) {      // nothing to do: no context is taken
        report_host_status(rout, ULMBLAS_GPU_OK, nullptr);
        return;
    }
    const int rc = with_context([&](HostContext &c) -> int {
        return gemm_host<T>(c, ta, tb, m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);
    });
    report_host_status(rout, rc, nullptr);
}

// interfaces/blas/F77/gemm.cc:149-195
int f77_info(const char *transA_, const char *transB_, int m, int n, int k,
             int ldA, int ldB, int ldC, bool &transA, bool &transB)
{
    const int a = toupper((unsigned char)*transA_);
    const int b = toupper((unsigned char)*transB_);
    transA = (a == 'T' || a == 'C');
    transB = (b == 'T' || b == 'C');
    const int numRowsA = (!transA) ? m : k;
    const int numRowsB = (!transB) ? k : n;
    if (a != 'N' && a != 'T' && a != 'C' && a != 'R') return 1;
    if (b != 'N' && b != 'T' && b != 'C' && b != 'R') return 2;
    if (m < 0) return 3;
    if (n < 0) return 4;
    if (k < 0) return 5;
    if (ldA < std::max(1, numRowsA)) return 8;
    if (ldB < std::max(1, numRowsB)) return 10;
    if (ldC < std::max(1, m)) return 13;
    return 0;
}

bool cblas_as_stored(int t) { return t == CblasNoTrans || t == AtlasConj; }
bool cblas_trans_valid(int t)
{
    return t == CblasNoTrans || t == CblasTrans || t == AtlasConj || t == CblasConjTrans;
}

// interfaces/blas/C/gemm.cc:410-466
int cblas_info(int order, int transA, int transB, int m, int n, int k, int ldA,
               int ldB, int ldC)
{
    int numRowsA, numRowsB;
    if (order == CblasColMajor) {
        numRowsA = cblas_as_stored(transA) ? m : k;
        numRowsB = cblas_as_stored(transB) ? k : n;
    } else {
        numRowsB = cblas_as_stored(transB) ? n : k;
        numRowsA = cblas_as_stored(transA) ? k : m;
    }
    if (order != CblasColMajor && order != CblasRowMajor) return 1;
    if (!cblas_trans_valid(transA)) return 2;
    if (!cblas_trans_valid(transB)) return 3;
    if (order == CblasColMajor) {
        if (m < 0) return 4;
        if (n < 0) return 5;
        if (k < 0) return 6;
        if (ldA < std::max(1, numRowsA)) return 9;
        if (ldB < std::max(1, numRowsB)) return 11;
        if (ldC < std::max(1, m)) return 14;
    } else {
        if (n < 0) return 4;
        if (m < 0) return 5;
        if (k < 0) return 6;
        if (ldB < std::max(1, numRowsB)) return 9;
        if (ldA < std::max(1, numRowsA)) return 11;
        if (ldC < std::max(1, n)) return 14;
    }
    return 0;
}

// the instantiations the other host sources link against
template int gemm_device<double>(bool, bool, int, int, int, double, const double *, int, const double *, int, double,
                                 double *, int, hipStream_t);
template int gemm_device<float>(bool, bool, int, int, int, float, const float *, int, const float *, int, float,
                                float *, int, hipStream_t);
template int launch_scale<double>(int, int, double, double *, int64_t, hipStream_t, int);
template int launch_scale<float>(int, int, float, float *, int64_t, hipStream_t, int);
template int gemm_tri_device<double>(int, bool, bool, int, int, double, const double *, int, const double *, int,
                                     double, double *, int, hipStream_t);
template int gemm_tri_device<float>(int, bool, bool, int, int, float, const float *, int, const float *, int, float,
                                    float *, int, hipStream_t);
template int copy_window<double>(void *, size_t, const void *, size_t, int, int, hipMemcpyKind, hipStream_t);
template int copy_window<float>(void *, size_t, const void *, size_t, int, int, hipMemcpyKind, hipStream_t);

}  // namespace ulmgpu

extern "C" {

void dgemm_(const char *transA_, const char *transB_, const int *m,
            const int *n, const int *k, const double *alpha, const double *A,
            const int *ldA, const double *B, const int *ldB,
            const double *beta, double *C, const int *ldC)
{
    bool ta, tb;
    int info = f77_info(transA_, transB_, *m, *n, *k, *ldA, *ldB, *ldC, ta, tb);
    if (info != 0) {
        xerbla_("DGEMM ", &info);
        return;
    }
    gemm_host_report<double>("dgemm_", ta, tb, *m, *n, *k, *alpha, A, *ldA, B,
                             *ldB, *beta, C, *ldC);
}

void sgemm_(const char *transA_, const char *transB_, const int *m,
            const int *n, const int *k, const float *alpha, const float *A,
            const int *ldA, const float *B, const int *ldB, const float *beta,
            float *C, const int *ldC)
{
    bool ta, tb;
    int info = f77_info(transA_, transB_, *m, *n, *k, *ldA, *ldB, *ldC, ta, tb);
    if (info != 0) {
        xerbla_("SGEMM ", &info);
        return;
    }
    gemm_host_report<float>("sgemm_", ta, tb, *m, *n, *k, *alpha, A, *ldA, B,
                            *ldB, *beta, C, *ldC);
}

void ulmblas_dgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB,
                   int m, int n, int k, double alpha, const double *A, int ldA,
                   const double *B, int ldB, double beta, double *C, int ldC)
{
    gemm_host_report<double>("ulmblas_dgemm", !cblas_as_stored(transA),
                             !cblas_as_stored(transB), m, n, k, alpha, A, ldA,
                             B, ldB, beta, C, ldC);
}

void ulmblas_sgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB,
                   int m, int n, int k, float alpha, const float *A, int ldA,
                   const float *B, int ldB, float beta, float *C, int ldC)
{
    gemm_host_report<float>("ulmblas_sgemm", !cblas_as_stored(transA),
                            !cblas_as_stored(transB), m, n, k, alpha, A, ldA, B,
                            ldB, beta, C, ldC);
}

void ATL_dgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB, int m,
               int n, int k, double alpha, const double *A, int ldA,
               const double *B, int ldB, double beta, double *C, int ldC)
{
    ulmblas_dgemm(transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);
}

void ATL_sgemm(enum CBLAS_TRANSPOSE transA, enum CBLAS_TRANSPOSE transB, int m,
               int n, int k, float alpha, const float *A, int ldA,
               const float *B, int ldB, float beta, float *C, int ldC)
{
    ulmblas_sgemm(transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);
}

void cblas_dgemm(enum CBLAS_ORDER order, enum CBLAS_TRANSPOSE transA,
                 enum CBLAS_TRANSPOSE transB, int m, int n, int k,
                 double alpha, const double *A, int ldA, const double *B,
                 int ldB, double beta, double *C, int ldC)
{
    int info = cblas_info(order, transA, transB, m, n, k, ldA, ldB, ldC);
    if (info != 0) {
        cblas_xerbla(info, "cblas_dgemm", "");
        return;
    }
    if (order == CblasColMajor) {
        ulmblas_dgemm(transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);
    } else {   // interfaces/blas/C/gemm.cc:478-484
        ulmblas_dgemm(transB, transA, n, m, k, alpha, B, ldB, A, ldA, beta, C, ldC);
    }
}

void cblas_sgemm(enum CBLAS_ORDER order, enum CBLAS_TRANSPOSE transA,
                 enum CBLAS_TRANSPOSE transB, int m, int n, int k, float alpha,
                 const float *A, int ldA, const float *B, int ldB, float beta,
                 float *C, int ldC)
{
    int info = cblas_info(order, transA, transB, m, n, k, ldA, ldB, ldC);
    if (info != 0) {
        cblas_xerbla(info, "cblas_sgemm", "");
        return;
    }
    if (order == CblasColMajor) {
        ulmblas_sgemm(transA, transB, m, n, k, alpha, A, ldA, B, ldB, beta, C, ldC);
    } else {
        ulmblas_sgemm(transB, transA, n, m, k, alpha, B, ldB, A, ldA, beta, C, ldC);
    }
}

int ulmblas_gpu_dgemm(int transA, int transB, int m, int n, int k,
                      double alpha, const double *dA, int ldA,
                      const double *dB, int ldB, double beta, double *dC,
                      int ldC, void *stream)
{
    return gemm_device<double>(transA != 0, transB != 0, m, n, k, alpha, dA,
                               ldA, dB, ldB, beta, dC, ldC,
                               static_cast<hipStream_t>(stream));
}

int ulmblas_gpu_sgemm(int transA, int transB, int m, int n, int k, float alpha,
                      const float *dA, int ldA, const float *dB, int ldB,
                      float beta, float *dC, int ldC, void *stream)
{
    return gemm_device<float>(transA != 0, transB != 0, m, n, k, alpha, dA, ldA,
                              dB, ldB, beta, dC, ldC,
                              static_cast<hipStream_t>(stream));
}

int ulmblas_gpu_test_control(int what, long value)
{
    switch (what) {
    case ULMBLAS_GPU_TEST_NARROW_LOADS:
        g_narrow_loads.store(value != 0);
        return ULMBLAS_GPU_OK;
    case ULMBLAS_GPU_TEST_LU_SPIN_LIMIT:
        lu_set_spin_limit(value);
        return ULMBLAS_GPU_OK;
    case ULMBLAS_GPU_TEST_SHARED_PIECES:
        if (value < -64 || value > 64) return ULMBLAS_GPU_BAD_ARGUMENT;
        g_sk_max_pieces.store((int)value);
        return ULMBLAS_GPU_OK;
    case ULMBLAS_GPU_TEST_SHARED_MUTE:
        g_sk_mute.store(value != 0);
        return ULMBLAS_GPU_OK;
    case ULMBLAS_GPU_TEST_SHARED_SPIN_LIMIT:
        g_sk_spin_limit.store(value >= 0 ? value : 1L << 20);
        return ULMBLAS_GPU_OK;
    case ULMBLAS_GPU_TEST_LU_SIMPLE_PANELS:
        lu_set_simple_panels(value != 0);
        return ULMBLAS_GPU_OK;
    case ULMBLAS_GPU_TEST_TRSM_PARTS:
        return trsm_set_parts((int)value);
    case ULMBLAS_GPU_TEST_HOST_HEAD:
        g_host_head.store((int)value);
        return ULMBLAS_GPU_OK;
    case ULMBLAS_GPU_TEST_TRI_WAY:
        if (value < 0 || value > 5) return ULMBLAS_GPU_BAD_ARGUMENT;
        g_tri_way.store((int)value);
        return ULMBLAS_GPU_OK;
    case ULMBLAS_GPU_TEST_WHOLE_C:
        g_whole_c.store(value < 0 ? -1 : (value != 0));
        return ULMBLAS_GPU_OK;
    case ULMBLAS_GPU_TEST_FAIL_ALLOC:
        g_fail_allocs.store(value);
        return ULMBLAS_GPU_OK;
    }
    return ULMBLAS_GPU_BAD_ARGUMENT;
}

int ulmblas_gpu_plan(int precision, int m, int n, int k, int reads_c, long ldA, long ldB, int out[4])
{
    if (m <= 0 || n <= 0 || k <= 0 || !out) return ULMBLAS_GPU_BAD_ARGUMENT;
    LaunchPlan p;
    if (precision == 'd') {
        const int f = g_forced_d.load();
        p = f > 0 ? plan_variant<double>(f, m, n, k, reads_c != 0, ldA, ldB) : choose_plan<double>(m, n, k, reads_c != 0, ldA, ldB);
    } else if (precision == 's') {
        const int f = g_forced_s.load();
        p = f > 0 ? plan_variant<float>(f, m, n, k, reads_c != 0, ldA, ldB) : choose_plan<float>(m, n, k, reads_c != 0, ldA, ldB);
    } else {
        return ULMBLAS_GPU_BAD_ARGUMENT;
    }
    out[0] = p.id;
    out[1] = p.whole_c ? 1 : 0;
    out[2] = p.share.groups;
    out[3] = p.share.tiles;
    return ULMBLAS_GPU_OK;
}

int ulmblas_gpu_device_status(void)
{
    SkDevice d;
    {
        int dev = -1;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
            (void)hipGetLastError();
            g_last_error = "no HIP device";
            return ULMBLAS_GPU_NO_DEVICE;
        }
        std::lock_guard<std::mutex> lock(g_sk_mu);
        d = g_sk_dev[dev];
    }
    if (!d.status) return ULMBLAS_GPU_OK;           // no launch on this device has shared a tile yet
    HIP_TRY(hipDeviceSynchronize());
    const unsigned word = take_status_word(0);
    g_shared_launches = 0;
    if (word == 0) return ULMBLAS_GPU_OK;
    g_last_error = std::to_string(word) + " bounded wait(s) of workgroups that shared a tile ran out since the last check; "
                   "what they would have added was computed by the launch that followed: the results are complete";
    return ULMBLAS_GPU_RECOVERED;
}

int ulmblas_gpu_set_variant(int precision, int variant)
{
    if (precision == 'd' && variant >= 0 && variant <= kNumD) {
        g_forced_d.store(variant);
        return ULMBLAS_GPU_OK;
    }
    if (precision == 's' && variant >= 0 && variant <= kNumS) {
        g_forced_s.store(variant);
        return ULMBLAS_GPU_OK;
    }
    return ULMBLAS_GPU_BAD_ARGUMENT;
}

const char *ulmblas_gpu_variant_name(int precision, int id)
{
    if (precision == 'd' && id >= 1 && id <= kNumD) return kVariantsD[id - 1].name;
    if (precision == 's' && id >= 1 && id <= kNumS) return kVariantsS[id - 1].name;
    return nullptr;
}

const char *ulmblas_gpu_last_error(void) { return g_last_error.c_str(); }

long ulmblas_gpu_alloc_count(void) { return g_host_allocs.load(); }

int ulmblas_gpu_last_status(void) { return g_last_status; }

void ulmblas_gpu_release(void)
{
    {
        // every context, each as soon as the call that holds it is over (calls that start meanwhile wait)
        std::unique_lock<std::mutex> lock(g_ctx_mu);
        for (int i = 0; i < kMaxContexts; ++i) {
            g_ctx_cv.wait(lock, [i] { return !g_ctx_busy[i]; });
            if (g_ctxs[i]) g_ctxs[i]->release();
        }
    }
    release_side_streams();
}

}  // extern "C"
