// Internals shared by the host-side sources of libulmblas_gpu: error state,
// the device-resident GEMM the other routines are built on, and the context
// of the host-pointer entry points (stream, cached device buffers, staging).
#ifndef ULMBLAS_GPU_INTERNAL_H
#define ULMBLAS_GPU_INTERNAL_H 1

#include "../../include/ulmblas_gpu.h"
#include "staging.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <deque>
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

// Whether the DMA engines can reach [p, p + bytes) directly: page-locked host
// memory known to the runtime (hipHostMalloc and the like).  Anything else,
// pageable memory included, is staged.
inline bool host_range_is_pinned(const void *p, size_t bytes)
{
    if (!p || bytes == 0) return false;
    const void *ends[2] = {p, static_cast<const char *>(p) + bytes - 1};
    for (const void *q : ends) {
        hipPointerAttribute_t attr;
        if (hipPointerGetAttributes(&attr, q) != hipSuccess) {
            (void)hipGetLastError();        // an unknown pointer is an answer here, not a failure
            return false;
        }
        if (attr.type != hipMemoryTypeHost) return false;
    }
    return true;
}

// Transfers of the host entry points' streamed paths: uploads on the context's
// h2d stream, downloads on its d2h stream, kernels in between on its compute
// stream, so that the three overlap.  Every transfer passes through the pinned
// rings in chunks that helper threads fill or drain (see staging.h); an operand
// that already lies in page-locked memory skips the rings and is copied where
// it lies.
template <typename T>
class Pipeline {
public:
    Pipeline(HostContext &c) : c_(c) {}

    // A window goes through the page-locked buffers in pieces of whole columns, a buffer's worth
    // each.  A call that moves only a few buffers' worth in all asks for finer pieces, a sixth of
    // the window (at least 4 MiB), so that the copy between the caller's memory and the buffers
    // and the transfer over the bus overlap there too (dgemm_ 2000^3: 5.1 -> 2.7 ms); calls that
    // keep several panels on their way lose by that (8192^3: 26.0 -> 27.2 ms).
    void set_fine(bool fine) { fine_ = fine; }
    size_t piece_bytes(size_t window_bytes) const
    {
        if (!fine_) return PinnedRing::kChunkBytes;
        return std::min<size_t>(PinnedRing::kChunkBytes, std::max<size_t>((size_t)4 << 20, window_bytes / 6));
    }

    // host window (rows x cols, pitch src_ld elements) -> device (pitch dst_ld)
    int upload(const T *src, size_t src_ld, T *dst, size_t dst_ld, size_t rows, size_t cols)
    {
        if (rows == 0 || cols == 0) return ULMBLAS_GPU_OK;
        const size_t row_bytes = rows * sizeof(T);
        if (host_range_is_pinned(src, ((cols - 1) * src_ld + rows) * sizeof(T))) {
            int rc = copy_window<T>(dst, dst_ld * sizeof(T), src, src_ld * sizeof(T), (int)rows, (int)cols,
                                    hipMemcpyHostToDevice, c_.h2d);
            if (rc) return rc;
            return pump(false);
        }
        const size_t per = std::max<size_t>(1, piece_bytes(row_bytes * cols) / row_bytes);
        for (size_t c0 = 0; c0 < cols; c0 += per) {
            const size_t nc = std::min(per, cols - c0);
            int slot;
            HIP_TRY(c_.in_ring.acquire(slot));
            copy_window_host(*c_.pool, c_.in_ring.ptr(slot), row_bytes,
                             reinterpret_cast<const char *>(src + c0 * src_ld), src_ld * sizeof(T), row_bytes, nc);
            if (dst_ld == rows) {
                HIP_TRY(hipMemcpyAsync(dst + c0 * dst_ld, c_.in_ring.ptr(slot), row_bytes * nc,
                                       hipMemcpyHostToDevice, c_.h2d));
            } else {
                HIP_TRY(hipMemcpy2DAsync(dst + c0 * dst_ld, dst_ld * sizeof(T), c_.in_ring.ptr(slot), row_bytes,
                                         row_bytes, nc, hipMemcpyHostToDevice, c_.h2d));
            }
            HIP_TRY(c_.in_ring.mark(slot, c_.h2d));
            int rc = pump(false);
            if (rc) return rc;
        }
        return ULMBLAS_GPU_OK;
    }

    // queue the download of a computed panel: device (pitch src_ld; 0: compact, pitch rows) -> host window
    void want_download(const T *src, T *dst, size_t dst_ld, size_t rows, size_t cols, hipEvent_t computed,
                       size_t src_ld = 0)
    {
        const size_t row_bytes = rows * sizeof(T);
        if (src_ld == 0) src_ld = rows;
        if (host_range_is_pinned(dst, ((cols - 1) * dst_ld + rows) * sizeof(T))) {
            Download d;
            d.src = src;
            d.src_ld = src_ld;
            d.dst = dst;
            d.dst_ld = dst_ld;
            d.row_bytes = row_bytes;
            d.cols = cols;
            d.after = computed;
            d.first = true;
            d.direct = true;
            waiting_.push_back(d);
            return;
        }
        const size_t per = std::max<size_t>(1, piece_bytes(row_bytes * cols) / row_bytes);
        for (size_t c0 = 0; c0 < cols; c0 += per) {
            Download d;
            d.src = src + c0 * src_ld;
            d.src_ld = src_ld;
            d.dst = dst + c0 * dst_ld;
            d.dst_ld = dst_ld;
            d.row_bytes = row_bytes;
            d.cols = std::min(per, cols - c0);
            d.after = computed;
            d.first = (c0 == 0);
            waiting_.push_back(d);
        }
    }

    // Move downloads along without blocking (block = false) or until all of
    // them have reached the caller's memory (block = true).
    int pump(bool block)
    {
        for (;;) {
            // results that have landed in a pinned buffer go to the caller's C
            while (!inflight_.empty()) {
                Download &d = inflight_.front();
                if (!block && hipEventQuery(ring_event_ready(d.slot)) != hipSuccess) break;
                HIP_TRY(c_.out_ring.wait(d.slot));
                copy_window_host(*c_.pool, reinterpret_cast<char *>(d.dst), d.dst_ld * sizeof(T),
                                 c_.out_ring.ptr(d.slot), d.row_bytes, d.row_bytes, d.cols);
                inflight_.pop_front();
                ++free_out_;
            }
            // computed panels are sent on their way while buffers are free
            while (!waiting_.empty() && (free_out_ > 0 || waiting_.front().direct)) {
                Download d = waiting_.front();
                waiting_.pop_front();
                if (d.first) HIP_TRY(hipStreamWaitEvent(c_.d2h, d.after, 0));
                if (d.direct) {     // straight into the caller's page-locked C; the final wait on the stream covers it
                    int rc = copy_window<T>(d.dst, d.dst_ld * sizeof(T), d.src, d.src_ld * sizeof(T),
                                            (int)(d.row_bytes / sizeof(T)), (int)d.cols, hipMemcpyDeviceToHost, c_.d2h);
                    if (rc) return rc;
                    continue;
                }
                HIP_TRY(c_.out_ring.acquire(d.slot));
                if (d.src_ld * sizeof(T) == d.row_bytes) {
                    HIP_TRY(hipMemcpyAsync(c_.out_ring.ptr(d.slot), d.src, d.row_bytes * d.cols,
                                           hipMemcpyDeviceToHost, c_.d2h));
                } else {
                    HIP_TRY(hipMemcpy2DAsync(c_.out_ring.ptr(d.slot), d.row_bytes, d.src, d.src_ld * sizeof(T),
                                             d.row_bytes, d.cols, hipMemcpyDeviceToHost, c_.d2h));
                }
                HIP_TRY(c_.out_ring.mark(d.slot, c_.d2h));
                --free_out_;
                inflight_.push_back(d);
            }
            if (!block || (waiting_.empty() && inflight_.empty())) return ULMBLAS_GPU_OK;
        }
    }

    void set_free_out(int n) { free_out_ = n; }

private:
    struct Download {
        const T *src;
        T *dst;
        size_t src_ld, dst_ld, row_bytes, cols;
        hipEvent_t after;
        bool first;
        bool direct = false;    // no ring buffer in between
        int slot = -1;
    };
    hipEvent_t ring_event_ready(int slot) { return c_.out_ring.event(slot); }

    HostContext &c_;
    std::deque<Download> waiting_, inflight_;
    int free_out_ = 0;
    bool fine_ = false;
};

// Whole windows for the host entry points that do not overlap transfers with
// kernels operand by operand: through the pinned rings where that pays (pageable
// memory then travels at the bus's rate instead of through the runtime's own
// staging), else as plain copies on the compute stream.
//
// Whether a call with this much to move, whose longest column is this long, takes the rings.
inline bool streams_transfers(HostContext &c, size_t bytes, size_t longest_col_bytes)
{
    return bytes >= ((size_t)16 << 20) && longest_col_bytes <= PinnedRing::kChunkBytes && c.ensure_pipeline();
}
// host -> device; kernels queued on the compute stream afterwards see the data
template <typename T>
int host_upload(HostContext &c, bool streamed, const T *src, size_t src_ld, T *dst, size_t dst_ld, size_t rows,
                size_t cols)
{
    if (!streamed) {
        return copy_window<T>(dst, dst_ld * sizeof(T), src, src_ld * sizeof(T), (int)rows, (int)cols,
                              hipMemcpyHostToDevice, c.stream);
    }
    Pipeline<T> pipe(c);
    pipe.set_fine(rows * cols * sizeof(T) <= 3 * PinnedRing::kChunkBytes);
    int rc = pipe.upload(src, src_ld, dst, dst_ld, rows, cols);
    if (rc) return rc;
    if ((rc = c.ensure_events(1))) return rc;
    HIP_TRY(hipEventRecord(c.events[0], c.h2d));
    HIP_TRY(hipStreamWaitEvent(c.stream, c.events[0], 0));
    return ULMBLAS_GPU_OK;
}
// device -> host, after everything queued on the compute stream so far; returns
// when the data is in the caller's memory
template <typename T>
int host_download(HostContext &c, bool streamed, const T *src, size_t src_ld, T *dst, size_t dst_ld, size_t rows,
                  size_t cols)
{
    if (rows == 0 || cols == 0) return ULMBLAS_GPU_OK;
    if (!streamed) {
        int rc = copy_window<T>(dst, dst_ld * sizeof(T), src, src_ld * sizeof(T), (int)rows, (int)cols,
                                hipMemcpyDeviceToHost, c.stream);
        if (rc) return rc;
        HIP_TRY(hipStreamSynchronize(c.stream));
        return ULMBLAS_GPU_OK;
    }
    int rc = c.ensure_events(2);
    if (rc) return rc;
    HIP_TRY(hipEventRecord(c.events[1], c.stream));
    Pipeline<T> pipe(c);
    pipe.set_free_out(c.out_ring.count());
    pipe.set_fine(rows * cols * sizeof(T) <= 3 * PinnedRing::kChunkBytes);
    pipe.want_download(src, dst, dst_ld, rows, cols, c.events[1], src_ld);
    if ((rc = pipe.pump(true))) return rc;
    HIP_TRY(hipStreamSynchronize(c.d2h));
    return ULMBLAS_GPU_OK;
}

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
