// Internals shared by the host-side sources of libulmblas_gpu: error state,
// the device-resident GEMM the other routines are built on, and the context
// of the host-pointer entry points (stream, cached device buffers, staging).
#ifndef ULMBLAS_GPU_INTERNAL_H
#define ULMBLAS_GPU_INTERNAL_H 1

#include "../../include/ulmblas_gpu.h"
#include "staging.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

namespace ulmgpu {

extern thread_local std::string g_last_error;
bool hip_ok(hipError_t e, const char *what);

#define HIP_TRY(expr)                                 \
    do {                                              \
        if (!::ulmgpu::hip_ok((expr), #expr)) return ULMBLAS_GPU_HIP_ERROR; \
    } while (0)

// C <- alpha*op(A)*op(B) + beta*C on device-resident column-major operands,
// enqueued on `stream` (gemm_host.hip; instantiated for double and float).
template <typename T>
int gemm_device(bool ta, bool tb, int m, int n, int k, T alpha, const T *dA,
                int ldA, const T *dB, int ldB, T beta, T *dC, int ldC,
                hipStream_t stream);

// While one of these lives, gemm_device calls of this thread launch the ragged
// strips of a product on the caller's stream instead of on side streams, and
// create no stream or event (for callers that may not allocate anything).
struct InlineStrips {
    InlineStrips();
    ~InlineStrips();
    InlineStrips(const InlineStrips &) = delete;
    InlineStrips &operator=(const InlineStrips &) = delete;
};

// B <- alpha*inv(op(A))*B (left) or alpha*B*inv(op(A)) (right), device-resident
// (trsm.hip; instantiated for double and float).
template <typename T>
int trsm_device(bool right, bool lower, bool trans, bool unit, int m, int n, T alpha, const T *dA, int ldA, T *dB,
                int ldB, hipStream_t stream);

// C <- beta*C on the m x n window (beta == 0 stores zeros without reading).
// tri: 0 = whole window, +1 = on and below the diagonal, -1 = on and above.
template <typename T>
int launch_scale(int m, int n, T beta, T *dC, int64_t ldC, hipStream_t stream, int tri = 0);

// One triangle (diagonal included) of the n x n block
// C <- alpha*op(A)*op(B) + beta*C; the rest of C is not touched.
template <typename T>
int gemm_tri_device(int tri, bool ta, bool tb, int n, int k, T alpha, const T *dA, int ldA, const T *dB, int ldB,
                    T beta, T *dC, int ldC, hipStream_t stream);

// Polls one wait of the LU panel kernel makes for the other workgroups before
// it gives up (negative: the default).  For tests of that path.
void lu_set_spin_limit(long polls);
// Testing: every LU panel takes the path of many small launches that wait for nobody.
void lu_set_simple_panels(bool on);
int trsm_set_parts(int parts);   // blocks of unknowns per launch of the triangular solve (testing)

// Copy the rows x cols window of a column-major matrix between host and
// device (pitches in bytes).
template <typename T>
int copy_window(void *dst, size_t dpitch, const void *src, size_t spitch,
                int rows, int cols, hipMemcpyKind kind, hipStream_t stream);

// ---------------------------------------------------------------------------
// host-pointer path: device operand buffers cached between calls (the role
// of the static MemoryPool in ulmblas/level3/gemm.tcc:50,57-58,85-86)
// ---------------------------------------------------------------------------
// Counters of all contexts together.
extern std::atomic<long> g_host_allocs;          // times a context went to the device allocator
extern std::atomic<long> g_fail_allocs;          // testing: this many allocations to come fail

struct HostContext {
    hipStream_t stream = nullptr;            // kernels
    hipStream_t h2d = nullptr, d2h = nullptr;
    void *buf[3] = {nullptr, nullptr, nullptr};
    size_t cap[3] = {0, 0, 0};
    // LU (lu.hip): pivots, exchange area + info word, transposed copy for the row-major entry
    int *lu_piv = nullptr;
    size_t lu_piv_cap = 0;
    void *lu_work = nullptr;
    int *lu_info = nullptr;
    void *lu_scratch = nullptr;
    size_t lu_scratch_cap = 0;
    // pipelined transfers
    std::unique_ptr<CopyPool> pool;
    PinnedRing in_ring, out_ring;
    std::vector<hipEvent_t> events;          // per-panel "uploaded" / "computed"
    bool pipeline_tried = false, pipeline_ok = false;

    int ensure_stream()
    {
        if (stream) return ULMBLAS_GPU_OK;
        int ndev = 0;
        if (hipGetDeviceCount(&ndev) != hipSuccess || ndev == 0) {
            g_last_error = "no HIP device";
            return ULMBLAS_GPU_NO_DEVICE;
        }
        HIP_TRY(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
        return ULMBLAS_GPU_OK;
    }
    // streams, pinned rings and helper threads of the pipelined path; if any of
    // it cannot be had the plain path below still serves every call
    bool ensure_pipeline()
    {
        if (pipeline_tried) return pipeline_ok;
        pipeline_tried = true;
        if (hipStreamCreateWithFlags(&h2d, hipStreamNonBlocking) != hipSuccess) return false;
        if (hipStreamCreateWithFlags(&d2h, hipStreamNonBlocking) != hipSuccess) return false;
        if (!in_ring.init(4) || !out_ring.init(4)) {
            in_ring.release();
            out_ring.release();
            (void)hipGetLastError();
            return false;
        }
        pool.reset(new CopyPool(staging_threads()));
        pipeline_ok = true;
        return true;
    }
    int ensure_events(size_t count)
    {
        while (events.size() < count) {
            hipEvent_t e;
            HIP_TRY(hipEventCreateWithFlags(&e, hipEventDisableTiming));
            events.push_back(e);
        }
        return ULMBLAS_GPU_OK;
    }
    // hipMalloc, counted, and failing on request (ULMBLAS_GPU_TEST_FAIL_ALLOC)
    static hipError_t device_alloc(void **p, size_t bytes)
    {
        if (g_fail_allocs.load() > 0) {
            g_fail_allocs.fetch_sub(1);
            return hipErrorOutOfMemory;
        }
        const hipError_t e = hipMalloc(p, bytes);
        if (e == hipSuccess) g_host_allocs.fetch_add(1);
        return e;
    }
    int reserve(int which, size_t bytes)
    {
        if (bytes <= cap[which]) return ULMBLAS_GPU_OK;
        if (buf[which]) {
            HIP_TRY(hipFree(buf[which]));
            buf[which] = nullptr;
            cap[which] = 0;
        }
        // grow with head-room so a sweep of rising sizes allocates rarely
        const size_t want = bytes + bytes / 4 + 4096;
        HIP_TRY(device_alloc(&buf[which], want));
        cap[which] = want;
        return ULMBLAS_GPU_OK;
    }
    void release()
    {
        for (int i = 0; i < 3; ++i) {
            if (buf[i]) (void)hipFree(buf[i]);
            buf[i] = nullptr;
            cap[i] = 0;
        }
        if (lu_piv) (void)hipFree(lu_piv);
        if (lu_work) (void)hipFree(lu_work);
        if (lu_scratch) (void)hipFree(lu_scratch);
        lu_piv = nullptr;
        lu_work = lu_scratch = nullptr;
        lu_info = nullptr;
        lu_piv_cap = lu_scratch_cap = 0;
    }
    // after a failed call: nothing of it may still be on its way when the caller gets its memory back
    void drain()
    {
        if (h2d) (void)hipStreamSynchronize(h2d);
        if (stream) (void)hipStreamSynchronize(stream);
        if (d2h) (void)hipStreamSynchronize(d2h);
        (void)hipGetLastError();
    }
};

// The host entry points work in a context each: a stream, cached device
// buffers, staging rings.  A call takes a free context for its duration
// (the one it had last time if that is free, so that a thread that repeats a
// shape finds its buffers), a new one if all are taken, up to kMaxContexts;
// beyond that it waits for one.  Calls from different threads therefore run
// side by side, as the reference's do (each takes its own pool blocks,
// ulmblas/auxiliary/memorypool.tcc:39-59).
constexpr int kMaxContexts = 4;
class ContextLease {
public:
    ContextLease();
    ~ContextLease();
    ContextLease(const ContextLease &) = delete;
    ContextLease &operator=(const ContextLease &) = delete;
    HostContext &get() { return *c_; }

private:
    HostContext *c_;
    int index_;
};

// Runs f(context) in a context of its own; if f fails, whatever it started is
// waited for before the context is given back.
template <class F>
int with_context(F &&f)
{
    ContextLease lease;
    HostContext &c = lease.get();
    const int rc = f(c);
    if (rc != ULMBLAS_GPU_OK) c.drain();
    return rc;
}

// The status of a host entry point's call, for ulmblas_gpu_last_status(), and
// on failure the error hook (the context's transfers are waited for first).
void report_host_status(const char *routine, int status, HostContext *c);

}  // namespace ulmgpu
#endif
